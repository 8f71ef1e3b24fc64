"""Parity of the HIP path (through ``ninetoothed_amd.make`` and the C ABI of
libnt_hip.so) with the CPU oracle on the same seeded inputs, at sizes the
oracle finishes in seconds, and with the torch ops the reference's own tests
compare against.  Bars: rtol = atol = 1e-2 for fp16 / bf16 (the reference's
tests/test_attention.py:102 states the same for fp16), 1e-5 for fp32 softmax."""

import functools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import ninetoothed_amd as ninetoothed
from ninetoothed_amd import Tensor, programs
from oracle import programs as oracle

pytestmark = pytest.mark.gpu

HALF_TOL = dict(rtol=1e-2, atol=1e-2)


def _native_only(kernel, expected_prefix):
    assert kernel.last_plan is not None and kernel.last_plan.startswith(expected_prefix), kernel.last_plan


def _randn(*shape, dtype=torch.float16, scale=1.0):
    return (torch.randn(*shape) * scale).to(dtype)


# ---- matmul ---------------------------------------------------------------


def _matmul_kernel(application=programs.matmul.application, **blocks):
    arrangement = functools.partial(programs.matmul.arrangement, **blocks) if blocks else programs.matmul.arrangement
    return ninetoothed.make(arrangement, application, (Tensor(2), Tensor(2), Tensor(2)))


@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (300, 200, 100), (64, 48, 8), (1, 1, 1), (257, 129, 65)))
def test_matmul_against_oracle(m, n, k):
    a, b = _randn(m, k), _randn(k, n)
    out = torch.empty(m, n, dtype=torch.float16, device="cuda")
    kernel = _matmul_kernel(programs.matmul.application_with_cast)
    kernel(a.cuda(), b.cuda(), out)
    _native_only(kernel, "launch_nt_matmul")
    expected = oracle.matmul(a.numpy(), b.numpy(), 64, 64, 64)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)
    assert torch.allclose(out, torch.matmul(a.cuda(), b.cuda()), **HALF_TOL)


def test_matmul_readme_program_fixed_blocks_and_strides():
    a, b = _randn(512, 384), _randn(384, 256)
    kernel = _matmul_kernel(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64)
    out = torch.empty(512, 256, dtype=torch.float16, device="cuda")
    kernel(a.cuda(), b.cuda(), out)
    assert torch.allclose(out, torch.matmul(a.cuda(), b.cuda()), **HALF_TOL)
    # column-major rhs, row-strided lhs, strided output
    bt = b.t().contiguous().cuda().t()
    wide = torch.zeros(512, 512, dtype=torch.float16, device="cuda")
    wide[:, :384] = a.cuda()
    out2 = torch.zeros(512, 512, dtype=torch.float16, device="cuda")
    kernel(wide[:, :384], bt, out2[:, ::2])
    assert torch.allclose(out2[:, ::2], out, rtol=0, atol=0)
    assert torch.count_nonzero(out2[:, 1::2]) == 0


def test_matmul_bfloat16_and_float32_output():
    a, b = _randn(256, 128, dtype=torch.bfloat16), _randn(128, 256, dtype=torch.bfloat16)
    kernel = _matmul_kernel()
    out = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
    kernel(a.cuda(), b.cuda(), out)
    expected = oracle.matmul(a.float().numpy(), b.float().numpy(), 64, 64, 64, out_dtype="bf16")
    # (two fp32 sums in different orders may round to neighbouring bf16 values: one ulp is at most 0.8 % of the value)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)
    assert torch.allclose(out.float(), a.cuda().float() @ b.cuda().float(), **HALF_TOL)
    out32 = torch.empty(256, 256, dtype=torch.float32, device="cuda")
    kernel(a.cuda(), b.cuda(), out32)
    assert torch.allclose(out32, a.cuda().float() @ b.cuda().float(), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (300, 200, 100), (64, 48, 8), (1, 1, 1), (257, 129, 65)))
def test_matmul_float32_operands(m, n, k):
    """fp32 tensors run on the fp32 MFMA (products and sums in fp32, no narrowing): against the oracle in
    fp32 and against torch at fp32 tolerances, contiguous and strided."""
    a, b = _randn(m, k, dtype=torch.float32), _randn(k, n, dtype=torch.float32)
    kernel = _matmul_kernel()
    out = torch.empty(m, n, dtype=torch.float32, device="cuda")
    kernel(a.cuda(), b.cuda(), out)
    _native_only(kernel, "launch_nt_matmul")
    expected = oracle.matmul(a.numpy(), b.numpy(), 64, 64, 64, out_dtype="fp32")
    assert np.allclose(out.cpu().numpy(), expected, rtol=1e-4, atol=1e-4)
    assert torch.allclose(out.cpu(), a.double().matmul(b.double()).float(), rtol=1e-4, atol=1e-4)
    out_t = torch.zeros(n, 2 * m, dtype=torch.float32, device="cuda")
    kernel(a.cuda(), b.t().contiguous().cuda().t(), out_t.t()[::2])
    assert torch.equal(out_t.t()[::2], out) and torch.count_nonzero(out_t.t()[1::2]) == 0


def test_addmm_float32_through_the_c_abi():
    from ninetoothed_amd import runtime

    lib = runtime.library()
    m, n, k = 200, 136, 72
    bias, a, b = (_randn(*shape, dtype=torch.float32).cuda() for shape in ((m, n), (m, k), (k, n)))
    out = torch.empty(m, n, dtype=torch.float32, device="cuda")
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(-1.25)
    fp32 = runtime.DATA_TYPE_INDEX["fp32"]
    runtime.check(lib.launch_nt_addmm(runtime.current_stream(), tensors[0], tensors[1], tensors[2], beta, alpha, tensors[3], fp32, 0, 0, 0))
    expected = 0.5 * bias.double() - 1.25 * (a.double() @ b.double())
    assert torch.allclose(out.double(), expected, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((4352, 4352, 2048), (4096, 4352, 2304), (4104, 4104, 2056)))
def test_products_a_few_tiles_over_whole_rounds_split_their_last_tile_rows(m, n, k, dtype):
    """17 x 17 (16 x 17) tiles of 256 x 256 on 256 CUs: the tile rows that fill a whole round run in one pass, the rows
    left over as a product of their own with the k range in parts.  Whole output of matmul and addmm against the
    program's arithmetic in fp32; block sizes keep the call in one pass, and both ways agree."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    a, b, bias = _randn(m, k, dtype=dtype).cuda(), _randn(k, n, dtype=dtype, scale=0.1).cuda(), _randn(m, n, dtype=dtype).cuda()
    out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (a, b, out, bias)]
    product = a.float() @ b.float()
    tolerance = dict(rtol=1e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-2, atol=2.0**-7 * float(product.abs().max()))
    runtime.check(lib.launch_nt_matmul(runtime.current_stream(), tensors[0], tensors[1], tensors[2], tag, tag, 0, 0, 0))
    assert "last rows with the k range in parts" in runtime.last_launch(), runtime.last_launch()
    assert torch.allclose(out.float(), product, **tolerance)
    in_parts = out.clone()
    out.fill_(float("nan"))
    runtime.check(lib.launch_nt_matmul(runtime.current_stream(), tensors[0], tensors[1], tensors[2], tag, tag, 256, 256, 32))
    assert "last rows" not in runtime.last_launch(), runtime.last_launch()
    assert torch.allclose(out.float(), in_parts.float(), **tolerance)
    top = (256 // ((n + 255) // 256)) * 256  # the rows of the one-pass part: the same kernel, the same bits
    assert torch.equal(out[:top], in_parts[:top])
    out.fill_(float("nan"))
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0)
    runtime.check(lib.launch_nt_addmm(runtime.current_stream(), tensors[3], tensors[0], tensors[1], beta, alpha, tensors[2], tag, 0, 0, 0))
    assert "last rows with the k range in parts" in runtime.last_launch(), runtime.last_launch()
    expected = 0.5 * bias.float() + 2.0 * product.to(dtype).float()
    wide = dict(rtol=1e-2, atol=tolerance["atol"] * 2.0 + 1e-2)  # (the product is rounded before it is doubled: two of its ulps)
    assert torch.allclose(out.float(), expected, **wide)


@pytest.mark.parametrize("m, n, k", ((128, 128, 4096), (100, 36, 5001), (1000, 1000, 1000), (512, 512, 512), (1, 7, 300)))
def test_float32_products_with_few_tiles_run_the_k_range_in_parts(m, n, k):
    """fp32 products of fewer than 192 tiles of 128 x 128 with at least 8 k tiles of 32: parts of the k range on
    workgroups of their own, partial tiles in scratch memory, then the sum and the addmm epilogue -- against float64,
    with operands and an output of any strides (the output inside a sentinel-filled buffer), as matmul and as addmm;
    block sizes keep the call on the one-pass kernel, and so does a captured graph on a stream without scratch."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    fp32 = runtime.DATA_TYPE_INDEX["fp32"]
    a = _randn(m, k, dtype=torch.float32).cuda()
    b_storage = _randn(n, k + 3, dtype=torch.float32).cuda()
    b = b_storage[:, 1 : k + 1].t()  # [k, n] stored by columns, rows off 16-byte boundaries
    bias = _randn(m, n, dtype=torch.float32).cuda()
    buffer = torch.full((m, 2 * n + 1), 7.0, dtype=torch.float32, device="cuda")
    out = buffer[:, 1::2]
    exact = a.double() @ b.double()
    tolerance = dict(rtol=1e-4, atol=1e-4 * max(1.0, (k / 512) ** 0.5))
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (a, b, out, bias)]
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(-1.25)
    in_parts = k >= 8 * 32

    runtime.check(lib.launch_nt_matmul(runtime.current_stream(), tensors[0], tensors[1], tensors[2], fp32, fp32, 0, 0, 0))
    assert ("k range in parts" in runtime.last_launch()) == in_parts, runtime.last_launch()
    assert torch.allclose(out.double(), exact, **tolerance)
    assert bool((buffer[:, 0::2] == 7.0).all())
    first = out.clone()
    runtime.check(lib.launch_nt_matmul(runtime.current_stream(), tensors[0], tensors[1], tensors[2], fp32, fp32, 128, 128, 32))
    assert "k range in parts" not in runtime.last_launch(), runtime.last_launch()
    assert torch.allclose(out.double(), exact, **tolerance)
    # (summing the k range in parts is the more accurate order)
    assert float((first.double() - exact).abs().max()) <= 2.0 * float((out.double() - exact).abs().max()) + 1e-6

    out.fill_(float("nan"))
    runtime.check(lib.launch_nt_addmm(runtime.current_stream(), tensors[3], tensors[0], tensors[1], beta, alpha, tensors[2], fp32, 0, 0, 0))
    assert ("k range in parts" in runtime.last_launch()) == in_parts, runtime.last_launch()
    assert torch.allclose(out.double(), 0.5 * bias.double() - 1.25 * exact, **tolerance)
    assert bool((buffer[:, 0::2] == 7.0).all())

    # captured on a stream that has no scratch buffer: one pass; replays checked
    torch.cuda.synchronize()
    lib.nt_release_workspaces()
    kernel = _matmul_kernel()
    plain = torch.empty(m, n, dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        kernel(a, b, plain)
        inside = runtime.last_launch()
    assert "k range in parts" not in inside, inside
    for replay in range(2):
        plain.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.allclose(plain.double(), exact, **tolerance), replay


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (1000, 768, 1024), (4096, 2048, 4096)))
def test_matmul_float32_output_on_the_fast_instances(m, n, k, dtype):
    """fp32 output of a plain product = the accumulators as they are; every instance that takes the
    shape has to write all of them (NaN-poisoned output, whole-output comparison with an fp32 product
    of the same rounded operands)."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    a = torch.randn(m, k, dtype=dtype, device="cuda")
    b = torch.randn(k, n, dtype=dtype, device="cuda")
    expected = a.float() @ b.float()
    kernel = _matmul_kernel()
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    kernel(a, b, out)
    assert torch.allclose(out, expected, rtol=1e-3, atol=1e-2 * (k / 512) ** 0.5)
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (a, b, out)]
    null = runtime.ArgumentTensor.null()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    served = 0
    for instance in range(lib.nt_gemm_num_configs()):
        out.fill_(float("nan"))
        result = lib.launch_nt_gemm_config(runtime.current_stream(), instance, null, tensors[0], tensors[1], null, null, tensors[2], tag, runtime.DATA_TYPE_INDEX["fp32"])
        if result == 1:
            continue
        assert result == 0
        served += 1
        assert torch.allclose(out, expected, rtol=1e-3, atol=1e-2 * (k / 512) ** 0.5), runtime.gemm_config_names()[instance]
    assert served >= 2


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (1000, 768, 1024), (4096, 2048, 4096)))
def test_transposed_rhs_on_the_fast_instances(m, n, k, dtype):
    """`x @ w.T` with `w` stored [N, K]: the rhs reaches the kernels with a unit k stride.  Every
    instance that takes it, matmul (both output types) and addmm, whole output, NaN-poisoned."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    a = torch.randn(m, k, dtype=dtype, device="cuda")
    w = torch.randn(n, k + 8, dtype=dtype, device="cuda")[:, :k]  # rows padded: a row stride that is not k
    b = w.t()
    bias = torch.randn(m, n, dtype=dtype, device="cuda")
    product = a.float() @ b.float()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    null = runtime.ArgumentTensor.null()
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0)
    # A plain product is held to rtol = atol = 1e-2 against the fp32 product of the same operands.  With a bias the
    # program rounds the product to the element type BEFORE it is scaled and added (tests/test_addmm.py:34-38 of the
    # reference): two correct fp32 sums that differ in their last bits may round to neighbouring values there, one
    # ulp of the product apart (bf16: up to 2^-7 of ~sqrt(k), times alpha = 2), and the bias may cancel the rest of
    # the value, so the absolute tolerance of that case follows the product's magnitude.
    biased = dict(rtol=2e-2, atol=2e-2 * (k / 512) ** 0.5) if dtype == torch.bfloat16 else dict(rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)
    for out_dtype, with_bias in ((dtype, False), (torch.float32, False), (dtype, True)):
        tolerance = biased if with_bias else HALF_TOL
        out = torch.empty(m, n, dtype=out_dtype, device="cuda")
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
        expected = 0.5 * bias.float() + 2.0 * product.to(dtype).float() if with_bias else product
        served = 0
        for instance in range(lib.nt_gemm_num_configs()):
            out.fill_(float("nan"))
            result = lib.launch_nt_gemm_config(
                runtime.current_stream(), instance, tensors[0] if with_bias else null, tensors[1], tensors[2], beta if with_bias else null,
                alpha if with_bias else null, tensors[3], tag, runtime.DATA_TYPE_INDEX["fp32" if out_dtype == torch.float32 else ("fp16" if dtype == torch.float16 else "bf16")],
            )
            if result == 1:
                continue
            assert result == 0
            served += 1
            assert torch.allclose(out.float(), expected, **tolerance), (runtime.gemm_config_names()[instance], out_dtype, with_bias)
        assert served >= 2
    # and through `make`
    out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    _matmul_kernel()(a, b, out)
    assert torch.allclose(out.float(), product, **HALF_TOL)


def _batched_matmul_kernel(application=programs.matmul.application, **blocks):
    arrangement = functools.partial(programs.matmul.batched_arrangement, **blocks) if blocks else programs.matmul.batched_arrangement
    return ninetoothed.make(arrangement, application, programs.matmul.batched_tensors())


@pytest.mark.parametrize("batch, m, n, k", ((3, 300, 200, 100), (2, 64, 48, 8), (5, 1, 1, 1), (4, 256, 256, 64)))
def test_batched_matmul_against_oracle(batch, m, n, k):
    """The matmul application under an arrangement with a leading batch dimension: every batch entry is the
    matmul program of the oracle; one launch of ``launch_nt_batched_matmul`` serves all of them."""
    a, b = _randn(batch, m, k), _randn(batch, k, n)
    out = torch.full((batch, m, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel = _batched_matmul_kernel()
    kernel(a.cuda(), b.cuda(), out)
    _native_only(kernel, "launch_nt_batched_matmul")
    expected = np.stack([oracle.matmul(a[i].numpy(), b[i].numpy(), 64, 64, 64) for i in range(batch)])
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_batched_matmul_layouts_and_output_types(dtype):
    from ninetoothed_amd import runtime

    batch, m, n, k = 12, 1024, 768, 512
    a, b = torch.randn(batch, m, k, dtype=dtype, device="cuda"), torch.randn(batch, k, n, dtype=dtype, device="cuda")
    product = torch.bmm(a.float(), b.float())
    kernel = _batched_matmul_kernel()
    out = torch.full((batch, m, n), float("nan"), dtype=dtype, device="cuda")
    kernel(a, b, out)
    assert torch.allclose(out.float(), product, **HALF_TOL)
    assert "any-stride" not in runtime.last_launch(), runtime.last_launch()  # dense operands: a direct-to-LDS instance
    # fp32 output, fixed blocks
    out32 = torch.full((batch, m, n), float("nan"), dtype=torch.float32, device="cuda")
    _batched_matmul_kernel(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64)(a, b, out32)
    assert torch.allclose(out32, product, rtol=1e-3, atol=1e-2)
    # rhs stored [batch, n, k] (`x @ w.transpose(1, 2)`), an lhs shared by every product, an output inside a wider buffer
    w = torch.randn(batch, n, k, dtype=dtype, device="cuda")
    shared = a[:1].expand(batch, m, k)
    wide = torch.full((batch, m, n + 8), 7.0, dtype=dtype, device="cuda")
    kernel(shared, w.transpose(1, 2), wide[:, :, :n])
    assert torch.allclose(wide[:, :, :n].float(), torch.bmm(shared.float(), w.transpose(1, 2).float()), **HALF_TOL)
    assert bool((wide[:, :, n:] == 7.0).all())
    # sizes that are no multiples of 8 and a batch order reversed by strides: the any-stride kernel, batch in the grid
    a2, b2 = torch.randn(5, 77, 45, dtype=dtype, device="cuda"), torch.randn(5, 45, 51, dtype=dtype, device="cuda")
    out2 = torch.full((5, 77, 51), float("nan"), dtype=dtype, device="cuda")
    kernel(a2.flip(0), b2, out2)
    assert torch.allclose(out2.float(), torch.bmm(a2.flip(0).float(), b2.float()), **HALF_TOL)
    assert "any-stride" in runtime.last_launch(), runtime.last_launch()
    # outputs of 197 x 197 elements each (no multiple of 8 between them) against k-contiguous operands: the instances
    # with tails, which then store element by element
    q4, k4 = torch.randn(24, 197, 64, dtype=dtype, device="cuda"), torch.randn(24, 197, 64, dtype=dtype, device="cuda")
    scores = torch.full((24, 197, 197), float("nan"), dtype=dtype, device="cuda")
    kernel(q4, k4.transpose(1, 2), scores)
    assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
    assert torch.allclose(scores.float(), torch.bmm(q4.float(), k4.float().transpose(1, 2)), **HALF_TOL)
    # larger products with such sizes run on dense copies, one per product -- also of an lhs that the products share
    a3, b3 = torch.randn(4, 300, 1001, dtype=dtype, device="cuda")[:, :, :1000], torch.randn(4, 1000, 500, dtype=dtype, device="cuda") * 0.1
    out3 = torch.full((4, 300, 504), 7.0, dtype=dtype, device="cuda")
    for lhs in (a3, a3[:1].expand(4, 300, 1000)):
        out3[:, :, :500] = float("nan")
        kernel(lhs, b3, out3[:, :, :500])
        assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
        assert torch.allclose(out3[:, :, :500].float(), torch.bmm(lhs.float(), b3.float()), rtol=1e-2, atol=1e-2 * 2**0.5)
        assert bool((out3[:, :, 500:] == 7.0).all())


def test_batched_matmul_float32_operands_and_empty_batches():
    a, b = torch.randn(3, 130, 70, device="cuda"), torch.randn(3, 70, 90, device="cuda")
    out = torch.full((3, 130, 90), float("nan"), device="cuda")
    kernel = _batched_matmul_kernel()
    kernel(a, b, out)
    assert torch.allclose(out, torch.bmm(a, b), rtol=1e-4, atol=1e-3)
    empty = torch.empty(0, 130, 90, device="cuda")
    kernel(a[:0], b[:0], empty)  # nothing to launch
    with pytest.raises(ninetoothed.UnsupportedProgram):
        kernel(a[:2], b, out)  # operands that disagree on the batch


def test_matmul_empty_and_errors():
    kernel = _matmul_kernel()
    out = torch.empty(0, 16, dtype=torch.float16, device="cuda")
    kernel(torch.empty(0, 8, dtype=torch.float16, device="cuda"), torch.empty(8, 16, dtype=torch.float16, device="cuda"), out)
    with pytest.raises(RuntimeError):
        kernel(torch.empty(4, 4, dtype=torch.float16), torch.empty(4, 4, dtype=torch.float16), torch.empty(4, 4, dtype=torch.float16))
    with pytest.raises(ninetoothed.UnsupportedProgram):
        kernel(*(torch.empty(4, 4, dtype=torch.float64, device="cuda") for _ in range(3)))


def test_matmul_large_properties():
    # 8192^3: linearity and an identity block, properties that hold at any size
    n = 8192
    a = _randn(n, n).cuda()
    b = _randn(n, n, scale=0.05).cuda()
    kernel = _matmul_kernel()
    out = torch.empty(n, n, dtype=torch.float16, device="cuda")
    kernel(a, b, out)
    _native_only(kernel, "launch_nt_matmul")
    rows = torch.randint(0, n, (64,), device="cuda")
    expected = (a[rows].float() @ b.float())
    assert torch.allclose(out[rows].float(), expected, **HALF_TOL)
    eye = torch.eye(n, dtype=torch.float16, device="cuda")
    kernel(a, eye, out)
    assert torch.equal(out, a)


# ---- addmm ----------------------------------------------------------------


def _addmm_kernel():
    return ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())


@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (100, 36, 52)))
def test_addmm_against_oracle(m, n, k):
    input, mat1, mat2 = _randn(m, n), _randn(m, k), _randn(k, n)
    beta, alpha = 0.37, 0.81
    out = torch.empty(m, n, dtype=torch.float16, device="cuda")
    kernel = _addmm_kernel()
    kernel(input.cuda(), mat1.cuda(), mat2.cuda(), beta, alpha, out)
    _native_only(kernel, "launch_nt_addmm")
    expected = oracle.addmm(input.numpy(), mat1.numpy(), mat2.numpy(), beta, alpha, 64, 64, 64)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)
    # the reference's own bar: tests/test_addmm.py:88-90, atol 0.075 against torch.addmm
    reference = torch.addmm(input.cuda(), mat1.cuda(), mat2.cuda(), beta=beta, alpha=alpha)
    assert torch.allclose(out, reference, atol=0.075)


def test_addmm_large():
    n = 8192
    input, mat1, mat2 = _randn(n, n).cuda(), _randn(n, n).cuda(), _randn(n, n, scale=0.05).cuda()
    out = torch.empty(n, n, dtype=torch.float16, device="cuda")
    kernel = _addmm_kernel()
    kernel(input, mat1, mat2, 0.5, 1.0, out)
    rows = torch.randint(0, n, (64,), device="cuda")
    expected = 0.5 * input[rows].float() + (mat1[rows].float() @ mat2.float()).half().float()
    assert torch.allclose(out[rows].float(), expected, **HALF_TOL)


# ---- softmax --------------------------------------------------------------


def _softmax(x, block_size=None):
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    out = torch.empty_like(x)
    kernel(x, out, BLOCK_SIZE=x.shape[-1] if block_size is None else block_size)
    _native_only(kernel, "launch_nt_softmax")
    return out


@pytest.mark.parametrize("m, n", ((1823, 781), (64, 4096), (5, 1), (3, 17000), (33, 8192)))
def test_softmax_against_oracle(m, n):
    x = torch.rand(m, n) if n == 781 else torch.randn(m, n)
    out = _softmax(x.cuda())
    assert np.allclose(out.cpu().numpy(), oracle.softmax(x.numpy()), rtol=1e-5, atol=1e-5)
    assert torch.allclose(out, torch.softmax(x.cuda(), dim=-1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", (torch.float32, torch.float16, torch.bfloat16))
@pytest.mark.parametrize(
    "m, n",
    ((100000, 32), (4099, 8), (7001, 64), (3000, 128), (513, 256), (1000, 1000), (128, 50257), (3, 200000), (9, 16385), (2, 70000),
     (3000, 29), (2000, 101), (700, 1001), (300, 4099), (50, 12289), (40, 7000)),
)
def test_softmax_short_rows_few_rows_and_long_rows(m, n, dtype):
    """Rows of a few vectors share a wave (8, 16 or 32 lanes each); few rows get a workgroup
    each; rows too long for registers take the two-sweep loop (running maximum and sum).
    The output lies in a sentinel-filled buffer with a row pitch of its own."""
    x = torch.randn(m, n, device="cuda").to(dtype)
    x[0, 0] = 30.0  # one dominant element
    if m > 1:
        x[1, n // 2 :] = float("-inf")  # a row whose second half is masked out
    pitch = n + (8 if n % 8 == 0 else 3)
    buffer = torch.full((m, pitch), 7.0, dtype=dtype, device="cuda")
    out = buffer[:, :n]
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    kernel(x, out, BLOCK_SIZE=1 << (n - 1).bit_length() if n > 1 else 1)
    _native_only(kernel, "launch_nt_softmax")
    expected = torch.softmax(x.float(), dim=-1)
    tolerance = {torch.float32: dict(rtol=1e-5, atol=1e-6), torch.float16: dict(rtol=2e-3, atol=1e-4), torch.bfloat16: dict(rtol=1.6e-2, atol=1e-3)}[dtype]
    assert torch.allclose(out.float(), expected, **tolerance)
    assert bool((buffer[:, n:] == 7.0).all())


@pytest.mark.parametrize("dtype", (torch.float32, torch.float16, torch.bfloat16))
@pytest.mark.parametrize("n", (1, 2, 3, 4, 5, 8, 10, 16, 17, 32))
def test_softmax_many_rows_of_a_few_elements(n, dtype):
    """Rows of up to 64 bytes, at least 4096 of them: one thread per row, fetched in the largest pieces that the
    row's bytes, the pitches and the addresses allow.  Input and output lie in sentinel-filled buffers with pitches
    of their own, once aligned and once one element off."""
    from ninetoothed_amd import runtime

    m = 5000
    tolerance = {torch.float32: dict(rtol=1e-5, atol=1e-6), torch.float16: dict(rtol=2e-3, atol=1e-4), torch.bfloat16: dict(rtol=1.6e-2, atol=1e-3)}[dtype]
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    for pitch, first in ((n, 0), (n + 8, 0), (n + 3, 1)):
        source = torch.full((m, pitch), float("inf"), dtype=dtype, device="cuda")
        x = source[:, first : first + n]
        x.copy_(torch.randn(m, n, device="cuda").to(dtype))
        x[0, 0] = 30.0
        if n > 1:
            x[1, n // 2 :] = float("-inf")
        buffer = torch.full((m, pitch), 7.0, dtype=dtype, device="cuda")
        out = buffer[:, first : first + n]
        kernel(x, out, BLOCK_SIZE=1 << (n - 1).bit_length() if n > 1 else 1)
        _native_only(kernel, "launch_nt_softmax")
        size = x.element_size()
        common = n * size | pitch * size | first * size  # every piece's offset and size is a multiple of its lowest set bit
        if n * size <= 64 and (common % 4 == 0 or (size == 2 and n <= 8)):
            assert "thread_per_row" in runtime.last_launch(), runtime.last_launch()
        assert torch.allclose(out.float(), torch.softmax(x.float(), dim=-1), **tolerance), (pitch, first)
        assert bool((buffer[:, :first] == 7.0).all()) and bool((buffer[:, first + n :] == 7.0).all())


def test_softmax_jit_decorator_form():
    # the decorator form with annotated parameters, as in the reference's tests/test_softmax.py:10-27
    import ninetoothed_amd.language as ntl
    from ninetoothed_amd import Symbol

    BLOCK_SIZE = Symbol("BLOCK_SIZE", constexpr=True)

    @ninetoothed.jit
    def softmax_kernel(
        input_row: Tensor(2, other=float("-inf")).tile((1, BLOCK_SIZE)),
        output_row: Tensor(2).tile((1, BLOCK_SIZE)),
    ):
        row_minus_max = input_row - ntl.max(input_row)
        numerator = ntl.exp(row_minus_max)
        denominator = ntl.sum(numerator)
        output_row = numerator / denominator  # noqa: F841

    x = torch.rand(1823, 781, device="cuda")
    out = torch.empty_like(x)
    softmax_kernel(x, out, BLOCK_SIZE=x.shape[-1])
    assert torch.allclose(out, torch.softmax(x, dim=-1))


def test_softmax_half_blocks_and_strides():
    x = torch.randn(128, 1000).to(torch.float16)
    out = _softmax(x.cuda())
    expected = torch.softmax(x.float(), dim=-1)
    assert torch.allclose(out.cpu().float(), expected, rtol=1e-2, atol=1e-3)
    y = torch.randn(16, 100)
    out = _softmax(y.cuda(), block_size=32)
    assert np.allclose(out.cpu().numpy(), oracle.softmax(y.numpy(), block_size=32), rtol=1e-5, atol=1e-6)
    wide = torch.randn(64, 512, device="cuda")
    view = wide[:, ::2]
    out = _softmax(view)
    assert torch.allclose(out, torch.softmax(view, dim=-1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", (torch.float32, torch.float16, torch.bfloat16))
def test_softmax_few_long_rows_are_cut_into_parts(dtype):
    """Up to 128 segments too long for the one-sweep kernels (or a handful that would leave most of the chip idle) are
    cut into parts: one launch for every part's maximum and sum, one that combines them and writes.  Checked: rows
    at an odd element offset in sentinel-filled buffers, a part that is all -inf, columns two elements apart,
    segments shorter than the row (against the oracle), a row of 2^24 elements (256 parts), and -- inside a captured
    graph on a stream that has no scratch buffer yet -- the fallback to one workgroup per segment."""
    from ninetoothed_amd import runtime

    tolerance = {torch.float32: dict(rtol=1e-5, atol=1e-7), torch.float16: dict(rtol=2e-3, atol=1e-6), torch.bfloat16: dict(rtol=1.6e-2, atol=1e-6)}[dtype]
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    for (m, n, first, step) in ((3, 200001, 1, 1), (16, 262144, 0, 1), (1, 1 << 24, 0, 1), (128, 50257, 3, 1), (5, 70000, 0, 2), (2, 40000, 1, 1)):
        pitch = first + n * step + 5
        source = torch.full((m, pitch), float("inf"), dtype=dtype, device="cuda")
        x = source[:, first : first + n * step : step]
        x.copy_(torch.randn(m, n, device="cuda").to(dtype))
        x[0, n - 1] = 12.0
        x[m - 1, 8192:20000] = float("-inf")  # a whole part (and more) without a finite element
        buffer = torch.full((m, pitch), 7.0, dtype=dtype, device="cuda")
        out = buffer[:, first : first + n * step : step]
        kernel(x, out, BLOCK_SIZE=1 << (n - 1).bit_length())
        _native_only(kernel, "launch_nt_softmax")
        assert "softmax_split" in runtime.last_launch(), (m, n, runtime.last_launch())
        expected = torch.softmax(x.float(), dim=-1)
        assert torch.allclose(out.float(), expected, **tolerance), (m, n, first, step)
        if n <= 300000:  # (a longer row's fp16 outputs are denormals or zeros)
            assert abs(float(out.float().sum(dim=-1).min()) - 1.0) < (1e-4 if dtype == torch.float32 else 2e-2)
        untouched = torch.ones_like(buffer, dtype=torch.bool)
        untouched[:, first : first + n * step : step] = False
        assert bool((buffer[untouched] == 7.0).all())
    if dtype == torch.float32:
        # segments of 2^17 elements of rows of 300000: each segment is a softmax of its own
        y = torch.randn(3, 300000)
        out = _softmax(y.cuda(), block_size=1 << 17)
        assert "softmax_split" in runtime.last_launch(), runtime.last_launch()
        assert np.allclose(out.cpu().numpy(), oracle.softmax(y.numpy(), block_size=1 << 17), rtol=1e-5, atol=1e-7)
    # under capture on a stream without a buffer for the parts: one workgroup per segment; afterwards, the parts
    x = torch.randn(4, 300000, device="cuda").to(dtype)
    out = torch.empty_like(x)
    expected = torch.softmax(x.float(), dim=-1)
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    runtime.library().nt_release_workspaces()  # (torch hands out its streams again and again: this one may have a buffer from an earlier test)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        kernel(x, out, BLOCK_SIZE=1 << 19)
        inside = runtime.last_launch()
    assert "softmax_loop_kernel" in inside, inside
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.allclose(out.float(), expected, **tolerance), replay
        with torch.cuda.stream(stream):
            kernel(x, out, BLOCK_SIZE=1 << 19)  # eager work between the replays: takes the buffer, runs in parts
        assert "softmax_split" in runtime.last_launch()
        torch.cuda.synchronize()
        assert torch.allclose(out.float(), expected, **tolerance), replay


def test_softmax_baseline_shape_properties():
    x = torch.randn(4096, 4096, device="cuda")
    out = _softmax(x)
    assert torch.allclose(out.sum(dim=-1), torch.ones(4096, device="cuda"), atol=1e-5)
    assert torch.allclose(out, _softmax(x + 2.5), rtol=1e-4, atol=1e-7)  # shift invariance
    assert torch.allclose(out, torch.softmax(x, dim=-1), rtol=1e-5, atol=1e-6)


# ---- attention ------------------------------------------------------------


def _attention(q, k, v, is_causal=False, scale=None):
    o = torch.full_like(q, float("nan"))
    if scale is None:
        kernel = ninetoothed.make(programs.attention.arrangement, programs.attention.application, programs.attention.tensors())
        kernel(q, k, v, is_causal, o)
    else:
        kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
        kernel(q, k, v, is_causal, scale, o)
    _native_only(kernel, "launch_nt_attention")
    return o


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("seq_len, emb_dim", ((160, 64), (1, 64), (100, 128), (333, 32)))
def test_attention_against_oracle(seq_len, emb_dim, is_causal):
    q, k, v = (_randn(2, 2, seq_len, emb_dim) for _ in range(3))
    out = _attention(q.cuda(), k.cuda(), v.cuda(), is_causal)
    expected = oracle.attention(q.numpy(), k.numpy(), v.numpy(), is_causal=is_causal, bm=64, bn=32)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("seq_len", (1024, 1))
def test_attention_reference_test_shapes(seq_len, is_causal):
    # reference: tests/test_attention.py:99-117 -- [2, 4, {1024, 1}, 64] fp16, scale 1, rtol = atol = 0.01
    q, k, v = (_randn(2, 4, seq_len, 64).cuda() for _ in range(3))
    out = _attention(q, k, v, is_causal)
    expected = F.scaled_dot_product_attention(q, k, v, is_causal=is_causal, scale=1)
    assert torch.allclose(out, expected, **HALF_TOL)


@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_scaled_head_dim_128_and_bfloat16(is_causal):
    q, k, v = (_randn(1, 3, 1000, 128).cuda() for _ in range(3))
    out = _attention(q, k, v, is_causal, scale=128**-0.5)
    expected = F.scaled_dot_product_attention(q, k, v, is_causal=is_causal, scale=128**-0.5)
    assert torch.allclose(out, expected, **HALF_TOL)
    qb, kb, vb = (t.to(torch.bfloat16) for t in (q, k, v))
    out = _attention(qb, kb, vb, is_causal, scale=128**-0.5)
    assert torch.allclose(out.float(), _attention_reference(qb, kb, vb, is_causal, 128**-0.5), **HALF_TOL)
    # (the stock bf16 operator rounds at other points: two bf16 roundings apart)
    expected = F.scaled_dot_product_attention(qb, kb, vb, is_causal=is_causal, scale=128**-0.5)
    assert torch.allclose(out.float(), expected.float(), rtol=3e-2, atol=3e-2)


def _attention_reference(q, k, v, is_causal, scale):
    """fp32 attention on the given (already rounded) operands."""
    scores = (q.float() * scale) @ k.float().transpose(-1, -2)
    if is_causal:
        mask = torch.ones(q.shape[-2], k.shape[-2], dtype=torch.bool, device=q.device).tril()
        scores = scores.masked_fill(~mask, float("-inf"))
    return torch.softmax(scores, dim=-1) @ v.float()


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16, torch.float32))
@pytest.mark.parametrize("emb_dim", (8, 40, 80, 96, 160, 192, 256))
def test_attention_other_head_dims(emb_dim, dtype, is_causal):
    """Head dimensions other than 32 / 64 / 128: 256 has a kernel of its own, other multiples of 8
    run on the next size up with the missing columns of Q, K and V read as zeros.  K and V lie
    inside larger Inf-filled rows, the output inside sentinel-filled ones: nothing past a row's
    end may be read into the result or written."""
    batch, heads, seq = 2, 3, 333
    pitch = emb_dim + 8
    def padded(fill):
        storage = torch.full((batch, heads, seq, pitch), fill, dtype=dtype, device="cuda")
        return storage, storage[..., :emb_dim]
    (_, q), (_, k), (_, v) = (padded(float("inf")) for _ in range(3))
    for t in (q, k, v):
        t.copy_(torch.randn(batch, heads, seq, emb_dim, device="cuda") * 0.5)
    o_storage, o = padded(7.0)
    o.fill_(float("nan"))
    scale = emb_dim**-0.5
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
    kernel(q, k, v, is_causal, scale, o)
    _native_only(kernel, "launch_nt_attention")
    expected = _attention_reference(q, k, v, is_causal, scale)
    assert torch.allclose(o.float(), expected, **HALF_TOL)
    assert bool((o_storage[..., emb_dim:] == 7.0).all())


@pytest.mark.parametrize("batch, heads, seq_q, seq_k, emb_dim", ((32, 32, 1, 2048, 128), (8, 32, 128, 8192, 128), (2, 8, 4096, 512, 64), (1, 8, 16, 65536, 128), (3, 5, 77, 1000, 64)))
@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_with_its_own_key_length(batch, heads, seq_q, seq_k, emb_dim, is_causal):
    """Queries against a longer (decoding, cross attention) or shorter key / value sequence; the
    causal mask keeps key j for query i when i >= j, counted from the start of both sequences."""
    q = _randn(batch, heads, seq_q, emb_dim).cuda()
    k, v = _randn(batch, heads, seq_k, emb_dim).cuda(), _randn(batch, heads, seq_k, emb_dim).cuda()
    o = torch.full_like(q, float("nan"))
    scale = emb_dim**-0.5
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
    kernel(q, k, v, is_causal, scale, o)
    _native_only(kernel, "launch_nt_attention")
    assert torch.allclose(o.float(), _attention_reference(q, k, v, is_causal, scale), **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("batch, heads, seq_q, seq_k, emb_dim", ((1, 32, 1, 32768, 128), (2, 4, 130, 5000, 64), (1, 2, 1024, 1024, 64), (1, 1, 300, 4097, 128), (3, 1, 7, 600, 64)))
def test_attention_split_key_range(batch, heads, seq_q, seq_k, emb_dim, is_causal, dtype):
    """Few (batch, head, query block) groups and many keys: parts of the key range run as
    workgroups of their own and a second kernel merges them.  With a causal mask, parts past
    the diagonal have no keys at all (the mask `q.offsets(-2) >= k.offsets(-2)` of the program,
    reference tests/test_attention.py:55, is aligned top-left whatever the two lengths are).
    Twice in a row on the same scratch memory."""
    q = _randn(batch, heads, seq_q, emb_dim).cuda().to(dtype)
    k, v = _randn(batch, heads, seq_k, emb_dim).cuda().to(dtype), _randn(batch, heads, seq_k, emb_dim).cuda().to(dtype)
    scale = emb_dim**-0.5
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
    expected = _attention_reference(q, k, v, is_causal, scale)
    for _ in range(2):
        o = torch.full_like(q, float("nan"))
        kernel(q, k, v, is_causal, scale, o)
        assert torch.allclose(o.float(), expected, **HALF_TOL)
    _native_only(kernel, "launch_nt_attention")


def test_attention_closed_forms_and_layouts():
    q, v = _randn(1, 2, 300, 64).cuda(), _randn(1, 2, 300, 64).cuda()
    k = torch.zeros_like(q)
    out = _attention(q, k, v)
    assert torch.allclose(out.float(), v.float().mean(dim=2, keepdim=True).expand_as(out), atol=5e-3)
    causal = _attention(q, k, v, True)
    assert torch.allclose(causal[:, :, 0], v[:, :, 0], atol=1e-3)
    # [batch, seq, heads, dim] storage viewed as [batch, heads, seq, dim]
    packed = _randn(2, 200, 3, 64).cuda()
    view = packed.permute(0, 2, 1, 3)
    out = _attention(view, view, view)
    expected = F.scaled_dot_product_attention(view, view, view, scale=1)
    assert torch.allclose(out, expected, **HALF_TOL)


@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_baseline_shape(is_causal):
    # every element of every (batch, head) is compared, on an output buffer that
    # starts as NaN, twice: a synchronisation mistake in the kernel shows up as a
    # few wrong rows in a few heads, not in every head
    q, k, v = (_randn(4, 32, 4096, 128).cuda() for _ in range(3))
    # fp32 attention on the same operands, eight heads at a time (the scores of one batch entry would take 2 GiB)
    expected = torch.cat([torch.cat([_attention_reference(q[b : b + 1, h : h + 8], k[b : b + 1, h : h + 8], v[b : b + 1, h : h + 8], is_causal, 128**-0.5)
                                     for h in range(0, 32, 8)], dim=1) for b in range(4)])
    vendor = torch.cat(
        [F.scaled_dot_product_attention(q[b : b + 1], k[b : b + 1], v[b : b + 1], is_causal=is_causal, scale=128**-0.5) for b in range(4)]
    )
    kernel = ninetoothed.make(
        programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True)
    )
    for _ in range(2):
        out = torch.full_like(q, float("nan"))
        kernel(q, k, v, is_causal, 128**-0.5, out)
        _native_only(kernel, "launch_nt_attention")
        assert torch.allclose(out.float(), expected, **HALF_TOL)
        assert torch.allclose(out, vendor, **HALF_TOL)  # the stock fp16 operator of the same GPU


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("emb_dim", (64, 128))
@pytest.mark.parametrize("block_size_m, block_size_n", ((0, 0), (256, 0), (0, 32), (0, 64)))
def test_attention_block_size_hints(block_size_m, block_size_n, emb_dim, is_causal):
    # the block sizes of the arrangement reach the library as hints that pick the
    # kernel variant; each variant is checked over the whole output, through the C ABI
    from ninetoothed_amd import runtime

    q, k, v = (_randn(2, 8, 2048 + 40, emb_dim).cuda() for _ in range(3))
    out = torch.full_like(q, float("nan"))
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (q, k, v, out)]
    code = runtime.library().launch_nt_attention(
        runtime.current_stream(), tensors[0], tensors[1], tensors[2],
        runtime.ArgumentTensor.from_scalar(int(is_causal)), runtime.ArgumentTensor.from_scalar(float(emb_dim**-0.5)),
        tensors[3], runtime.DATA_TYPE_INDEX["fp16"], block_size_m, block_size_n,
    )
    assert code == 0
    expected = F.scaled_dot_product_attention(q, k, v, is_causal=is_causal, scale=emb_dim**-0.5)
    assert torch.allclose(out, expected, **HALF_TOL)


@pytest.mark.parametrize("emb_dim", (64, 128))
@pytest.mark.parametrize("batch, heads, seq_q, seq_k", ((8, 32, 300, 333), (8, 32, 600, 200), (2, 16, 1100, 1500), (1, 8, 2048 + 17, 2048 + 17)))
def test_attention_causal_waves_stop_at_their_last_key_block(batch, heads, seq_q, seq_k, emb_dim):
    # with a causal mask the waves of a workgroup need different numbers of key blocks (the ones with the upper
    # query rows fewer); they leave the block loop at different steps but keep loading and synchronising:
    # ragged ends, more and fewer keys than queries, few and many query blocks
    q = _randn(batch, heads, seq_q, emb_dim).cuda()
    k, v = (_randn(batch, heads, seq_k, emb_dim).cuda() for _ in range(2))
    kernel = ninetoothed.make(
        programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True)
    )
    expected = _attention_reference(q, k, v, True, emb_dim**-0.5)
    for _ in range(2):
        out = torch.full_like(q, float("nan"))
        kernel(q, k, v, True, emb_dim**-0.5, out)
        assert torch.allclose(out.float(), expected, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("emb_dim", (64, 128))
def test_attention_many_short_sequences(emb_dim, dtype):
    # enough 256-row query blocks for the eight-wave loop (512 of them), with ragged ends on both
    # the query side (300 = 256 + 44) and the key side (333), and keys of another length than queries
    q = _randn(8, 32, 300, emb_dim, dtype=dtype).cuda()
    k, v = (_randn(8, 32, 333, emb_dim, dtype=dtype).cuda() for _ in range(2))
    kernel = ninetoothed.make(
        programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True)
    )
    expected = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), scale=emb_dim**-0.5)
    for _ in range(2):
        out = torch.full_like(q, float("nan"))
        kernel(q, k, v, False, emb_dim**-0.5, out)
        _native_only(kernel, "launch_nt_attention")
        assert torch.allclose(out.float(), expected, **HALF_TOL)


# ---- conv2d ---------------------------------------------------------------


def _conv2d(x, w, padding, application=programs.conv2d.application):
    n, _, h, width = x.shape
    k, _, r, s = w.shape
    p, q = h + 2 * padding[0] - r + 1, width + 2 * padding[1] - s + 1
    out = torch.empty(n, k, p, q, dtype=x.dtype, device=x.device)
    kernel = ninetoothed.make(programs.conv2d.arrangement, application, programs.conv2d.tensors())
    kernel(x, w, out, padding_h=padding[0], padding_w=padding[1])
    _native_only(kernel, "launch_nt_conv2d")
    return out


@pytest.mark.parametrize("padding", ((0, 0), (1, 1), (0, 1), (2, 0)))
def test_conv2d_against_oracle(padding):
    x = torch.rand(2, 6, 9, 8).to(torch.float16)
    w = torch.rand(5, 6, 3, 3).to(torch.float16)
    out = _conv2d(x.cuda(), w.cuda(), padding)
    expected = oracle.conv2d(x.numpy(), w.numpy(), padding=padding, bm=16, bn=4, bk=8)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)


@pytest.mark.parametrize("padding", ((0, 0), (1, 1), (2, 0)))
def test_conv2d_float32_tensors(padding):
    # (the accumulator is stored as it is: the reference's conv2d application rounds it to fp16 first)
    application = programs.matmul.application
    x = torch.rand(2, 6, 9, 8)
    w = torch.rand(5, 6, 3, 3)
    with pytest.raises(ninetoothed.UnsupportedProgram):
        _conv2d(x.cuda(), w.cuda(), padding)
    out = _conv2d(x.cuda(), w.cuda(), padding, application)
    assert out.dtype == torch.float32
    expected = oracle.conv2d(x.numpy(), w.numpy(), padding=padding, bm=16, bn=4, bk=8, dtype="fp32")
    assert np.allclose(out.cpu().numpy(), expected, rtol=1e-4, atol=1e-4)
    big_x, big_w = torch.randn(3, 32, 20, 24, device="cuda"), torch.randn(48, 32, 3, 3, device="cuda")
    assert torch.allclose(_conv2d(big_x, big_w, padding, application).cpu(), F.conv2d(big_x.cpu().double(), big_w.cpu().double(), padding=padding).float(), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("padding", ((0, 0), (1, 1), (0, 1), (2, 0)))
def test_conv2d_reference_test_shapes(padding):
    # reference: tests/test_conv2d.py:116-133 -- N4 C64 H16 W16 K512 R3 S3, torch.rand, rtol = atol = 1e-3
    x = torch.rand(4, 64, 16, 16, dtype=torch.float16, device="cuda")
    w = torch.rand(512, 64, 3, 3, dtype=torch.float16, device="cuda")
    out = _conv2d(x, w, padding)
    expected = F.conv2d(x, w, padding=padding)
    assert torch.allclose(out, expected, rtol=1e-3, atol=1e-3)


def test_conv2d_baseline_shape_and_1x1():
    x = _randn(32, 256, 56, 56, scale=0.1).cuda()
    w = _randn(256, 256, 3, 3, scale=0.1).cuda()
    out = _conv2d(x, w, (1, 1))
    expected = F.conv2d(x[:2], w, padding=1)
    assert torch.allclose(out[:2], expected, **HALF_TOL)
    w1 = _randn(64, 256, 1, 1, scale=0.1).cuda()
    out = _conv2d(x[:1], w1, (0, 0))
    as_matmul = (x[:1].permute(0, 2, 3, 1).reshape(-1, 256).float() @ w1.reshape(64, 256).t().float()).reshape(1, 56, 56, 64).permute(0, 3, 1, 2)
    assert torch.allclose(out.float(), as_matmul, **HALF_TOL)


@pytest.mark.parametrize(
    "n, c, h, w, k, r, s, padding",
    (
        (4, 64, 56, 56, 64, 3, 3, (1, 1)),     # 64 output channels: 128 x 64 tiles
        (4, 128, 28, 28, 128, 3, 3, (1, 1)),
        (8, 256, 14, 14, 256, 3, 3, (1, 1)),   # 196 positions per image: tiles span images, P*Q % 8 != 0
        (8, 512, 7, 7, 512, 3, 3, (1, 1)),     # 49 positions per image
        (5, 64, 56, 56, 256, 1, 1, (0, 0)),
        (16, 256, 28, 28, 128, 3, 3, (1, 1)),  # 256 x 128 tiles
        (2, 320, 16, 16, 320, 3, 3, (1, 1)),
        (3, 32, 9, 11, 192, 3, 2, (1, 0)),     # odd sizes all round
        (40, 96, 7, 5, 64, 2, 3, (0, 2)),
        (4, 3, 64, 64, 64, 7, 7, (3, 3)),      # channels padded to the k step of 32: a stem convolution
        (4, 16, 20, 20, 128, 3, 3, (1, 1)),
        (3, 40, 12, 12, 64, 3, 3, (1, 1)),
        (2, 200, 9, 9, 64, 1, 1, (0, 0)),
        (4, 64, 16, 16, 96, 3, 3, (1, 1)),     # partial last tiles of output channels
        (4, 32, 32, 32, 24, 3, 3, (1, 1)),
        (16, 64, 32, 32, 1000, 1, 1, (0, 0)),
        (2, 64, 20, 20, 328, 3, 3, (1, 1)),
    ),
)
def test_conv2d_layer_shapes_on_the_direct_to_lds_path(n, c, h, w, k, r, s, padding):
    """Layers other than the baseline's stay on the implicit-GEMM kernel: fewer output channels
    (narrower tiles), small images (GEMM rows run across images, stores element by element when
    P*Q is not a multiple of 8).  Whole NaN-poisoned output against an fp32 convolution of the
    same rounded operands (MIOpen's own half kernels deviate by more than the tolerance)."""
    dtype = torch.float16  # the program rounds its product to float16 (tests/test_conv2d.py:44-48)
    x = (torch.randn(n, c, h, w, device="cuda") * 0.5).to(dtype)
    weight = (torch.randn(k, c, r, s, device="cuda") * 0.1).to(dtype)
    p_out, q_out = h + 2 * padding[0] - r + 1, w + 2 * padding[1] - s + 1
    guard = torch.full((n * k * p_out * q_out + 64,), 7.0, dtype=dtype, device="cuda")
    out = guard[: n * k * p_out * q_out].view(n, k, p_out, q_out)
    out.fill_(float("nan"))
    kernel = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    kernel(x, weight, out, padding_h=padding[0], padding_w=padding[1])
    assert "implicit" in kernel.last_plan or "gemm" in kernel.last_plan
    expected = F.conv2d(x.float(), weight.float(), padding=padding)
    assert torch.allclose(out.float(), expected, rtol=1e-2, atol=1e-2)
    assert bool((guard[n * k * p_out * q_out :] == 7.0).all())


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize(
    "n, c, h, w, k, r, s, padding",
    (
        (2, 32, 8, 8, 256, 3, 3, (1, 1)),      # one tile that holds the tensor's first and last rows
        (1, 32, 16, 24, 256, 3, 3, (1, 1)),
        (3, 64, 24, 40, 256, 3, 3, (1, 1)),
        (4, 64, 28, 32, 256, 3, 3, (1, 1)),    # 14 tiles
        (2, 32, 10, 18, 256, 3, 3, (0, 0)),    # no padding
        (2, 32, 8, 16, 256, 3, 3, (2, 1)),     # two rows of padding above and below
        (2, 32, 12, 18, 512, 5, 5, (2, 1)),    # taps repeat after 25 tiles
        (2, 64, 10, 16, 256, 1, 1, (0, 0)),
        (2, 32, 9, 17, 256, 2, 2, (0, 0)),
        (2, 16, 12, 9, 424, 3, 2, (1, 0)),     # a partial second tile of output channels, input rows of 9 pixels
        (5, 96, 14, 8, 256, 3, 3, (1, 1)),     # image rows of one piece: every piece is at both borders
    ),
)
def test_conv2d_one_launch_path(n, c, h, w, k, r, s, padding, dtype):
    """launch_nt_conv2d with block_size_m = 3 (the tensors as they lie, no scratch memory), whole output against an
    fp32 convolution of the same operands.  The input is a channel slice of a larger Inf-filled tensor, so a
    load that strays outside an image's rows, or is not cleared at a border, shows up."""
    from ninetoothed_amd import runtime

    big = torch.full((n, c + 2, h, w), float("inf"), dtype=dtype, device="cuda")
    x = big[:, 1 : c + 1]
    x.copy_((torch.randn(n, c, h, w, device="cuda") * 0.5).to(dtype))
    weight = (torch.randn(k, c, r, s, device="cuda") * 0.1).to(dtype)
    p_out, q_out = h + 2 * padding[0] - r + 1, w + 2 * padding[1] - s + 1
    guard = torch.full((n * k * p_out * q_out + 64,), 7.0, dtype=dtype, device="cuda")
    out = guard[: n * k * p_out * q_out].view(n, k, p_out, q_out)
    out.fill_(float("nan"))
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, out)]
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, tag, padding[0], padding[1], 3, 0, 0) == 0
    expected = F.conv2d(x.float(), weight.float(), padding=padding)
    assert torch.allclose(out.float(), expected, **HALF_TOL)
    assert bool((guard[n * k * p_out * q_out :] == 7.0).all())


def _conv2d_with_steps(x, w, padding, stride, dilation, floor_mode=True, **blocks):
    n, _, h, width = x.shape
    k, _, r, s = w.shape

    def windows(size, pad, taps, spacing, step):
        span = size + 2 * pad - spacing * (taps - 1) - 1
        return span // step + 1 if floor_mode else -(-span // step) + 1

    p, q = windows(h, padding[0], r, dilation[0], stride[0]), windows(width, padding[1], s, dilation[1], stride[1])
    out = torch.full((n, k, p, q), float("nan"), dtype=x.dtype, device=x.device)
    arrangement = functools.partial(programs.conv2d.arrangement, stride=stride, dilation=dilation, floor_mode=floor_mode, **blocks)
    kernel = ninetoothed.make(arrangement, programs.conv2d.application, programs.conv2d.tensors())
    kernel(x, w, out, padding_h=padding[0], padding_w=padding[1])
    _native_only(kernel, "launch_nt_conv2d")
    return out, kernel


@pytest.mark.parametrize("floor_mode", (True, False))
@pytest.mark.parametrize("stride, dilation, padding", (((2, 2), (1, 1), (1, 1)), ((1, 2), (2, 1), (0, 1)), ((3, 1), (1, 2), (2, 2))))
def test_conv2d_with_stride_and_dilation_against_oracle(stride, dilation, padding, floor_mode):
    """`tile(..., strides, dilation)` in the conv2d arrangement (reference src/ninetoothed/tensor.py:199-286): the
    HIP path against the oracle's arrangement-driven execution, both roundings of the number of windows."""
    x = (torch.rand(2, 8, 11, 10) - 0.5).to(torch.float16)
    w = (torch.rand(16, 8, 3, 2) - 0.5).to(torch.float16)
    out, kernel = _conv2d_with_steps(x.cuda(), w.cuda(), padding, stride, dilation, floor_mode)
    expected = oracle.conv2d(x.numpy(), w.numpy(), padding=padding, bm=32, bn=16, bk=16, stride=stride, dilation=dilation, floor_mode=floor_mode)
    assert out.shape == expected.shape
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)
    if stride != (1, 1) or dilation != (1, 1):
        assert kernel.last_plan.startswith("launch_nt_conv2d_strided")


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16, torch.float32))
@pytest.mark.parametrize(
    "n, c, h, w, k, r, s, padding, stride, dilation",
    (
        (8, 64, 56, 56, 128, 3, 3, (1, 1), (2, 2), (1, 1)),   # a down-sampling layer
        (4, 256, 28, 28, 256, 3, 3, (2, 2), (1, 1), (2, 2)),  # a dilated layer
        (4, 128, 30, 30, 256, 1, 1, (0, 0), (2, 2), (1, 1)),  # 1 x 1 with stride: not the batched product
        (2, 3, 64, 64, 32, 7, 7, (3, 3), (2, 2), (1, 1)),     # a stem layer on three channels
        (3, 20, 19, 23, 24, 3, 5, (1, 2), (2, 3), (2, 1)),
    ),
)
def test_conv2d_with_stride_and_dilation_layer_shapes(n, c, h, w, k, r, s, padding, stride, dilation, dtype):
    from ninetoothed_amd import runtime

    x = _randn(n, c, h, w, dtype=dtype, scale=0.2).cuda()
    weight = _randn(k, c, r, s, dtype=dtype, scale=0.2).cuda()
    application = {torch.float16: programs.conv2d.application, torch.bfloat16: programs.matmul.application_with_bfloat16_cast, torch.float32: programs.matmul.application}[dtype]
    expected = F.conv2d(x.float(), weight.float(), padding=padding, stride=stride, dilation=dilation)
    out = torch.full(expected.shape, float("nan"), dtype=dtype, device="cuda")
    arrangement = functools.partial(programs.conv2d.arrangement, stride=stride, dilation=dilation, floor_mode=True)
    kernel = ninetoothed.make(arrangement, application, programs.conv2d.tensors())
    for _ in range(2):
        kernel(x, weight, out, padding_h=padding[0], padding_w=padding[1])
    assert kernel.last_plan.startswith("launch_nt_conv2d_strided"), kernel.last_plan
    tolerance = dict(rtol=1e-3, atol=1e-3) if dtype == torch.float32 else HALF_TOL
    assert torch.allclose(out.float(), expected, **tolerance), float((out.float() - expected).abs().max())
    if dtype != torch.float32 and k % 8 == 0 and c >= 2 and n * expected.shape[2] * expected.shape[3] >= 1024:
        assert runtime.last_launch().startswith("conv2d path 2"), runtime.last_launch()  # the repacking way takes these
    # each way by name through the C ABI
    tag = runtime.DATA_TYPE_INDEX[{torch.float16: "fp16", torch.bfloat16: "bf16", torch.float32: "fp32"}[dtype]]
    for path in (1, 2):
        y = torch.full_like(out, float("nan"))
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
        assert runtime.library().launch_nt_conv2d_strided(runtime.current_stream(), *tensors, tag, *padding, *stride, *dilation, path, 0, 0) == 0
        assert torch.allclose(y.float(), expected, **tolerance), path
    # an output of another size is refused
    y = torch.empty(n, k, expected.shape[2] + 2, expected.shape[3], dtype=dtype, device="cuda")
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
    assert runtime.library().launch_nt_conv2d_strided(runtime.current_stream(), *tensors, tag, *padding, *stride, *dilation, 0, 0, 0) == 1  # hipErrorInvalidValue


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("channels", (2, 3, 4, 8, 9, 13, 16, 17))
def test_conv2d_few_input_channels_on_the_repacked_path(channels, dtype):
    """Up to 16 input channels are padded to 8 or 16, not 32, on the repacked path: a k step then holds 4 or 2 filter
    taps, the last step of a filter whose taps do not fill it reads zeros (7 x 7 = 49 taps, 3 x 5 = 15)."""
    from ninetoothed_amd import runtime

    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    for (n, h, w, k, r, s_, padding, stride, dilation) in ((3, 40, 36, 64, 7, 7, (3, 3), (2, 2), (1, 1)), (2, 33, 31, 24, 3, 5, (1, 2), (1, 1), (2, 1)), (2, 32, 32, 40, 1, 1, (0, 0), (1, 1), (1, 1))):
        x = _randn(n, channels, h, w, dtype=dtype, scale=0.3).cuda()
        weight = _randn(k, channels, r, s_, dtype=dtype, scale=0.3).cuda()
        expected = F.conv2d(x.float(), weight.float(), padding=padding, stride=stride, dilation=dilation)
        y = torch.full(expected.shape, float("nan"), dtype=dtype, device="cuda")
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
        if stride == (1, 1) and dilation == (1, 1):
            assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, tag, *padding, 2, 0, 0) == 0
        else:
            assert runtime.library().launch_nt_conv2d_strided(runtime.current_stream(), *tensors, tag, *padding, *stride, *dilation, 2, 0, 0) == 0
        assert runtime.last_launch().startswith("conv2d path 2"), runtime.last_launch()
        assert torch.allclose(y.float(), expected, **HALF_TOL), (channels, r, s_, float((y.float() - expected).abs().max()))


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("channels", (3, 20, 32, 64, 72))
def test_conv2d_channels_last_and_sliced_tensors_on_the_repacked_path(channels, dtype):
    """Channels-last inputs are read in place when their channels fill whole k steps (32, 64) and copied by rows of
    channels otherwise; outputs that are no contiguous NCHW tensor (channels last, a window of a wider buffer whose
    other elements must stay as they were) are stored element by element."""
    from ninetoothed_amd import runtime

    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    for (n, h, w, k, r, s_, padding) in ((3, 20, 18, 40, 3, 3, (1, 1)), (2, 15, 17, 64, 1, 1, (0, 0)), (2, 16, 16, 24, 5, 3, (2, 0))):
        x = _randn(n, channels, h, w, dtype=dtype, scale=0.3).cuda()
        weight = _randn(k, channels, r, s_, dtype=dtype, scale=0.3).cuda()
        expected = F.conv2d(x.float(), weight.float(), padding=padding)
        p, q = expected.shape[2:]
        x_last = x.to(memory_format=torch.channels_last)
        assert x_last.stride(1) == 1
        wide = torch.full((n, k + 3, p + 2, q + 5), 7.0, dtype=dtype, device="cuda")
        window = wide[:, 2 : 2 + k, 1 : 1 + p, 3 : 3 + q]
        planes = torch.full((n, channels, h * w + 3), float("inf"), dtype=dtype, device="cuda")
        x_odd = planes[:, :, 1 : 1 + h * w].view(n, channels, h, w)  # NCHW whose channel planes start at odd elements
        x_odd.copy_(x)
        outputs = (
            (x_odd, weight, torch.full(expected.shape, float("nan"), dtype=dtype, device="cuda")),
            (x_last, weight.to(memory_format=torch.channels_last), torch.full(expected.shape, float("nan"), dtype=dtype, device="cuda").to(memory_format=torch.channels_last)),
            (x_last, weight, torch.full(expected.shape, float("nan"), dtype=dtype, device="cuda")),
            (x, weight, window),
            (x_last[:, :, :, 1:], weight, None),  # a channels-last input that is not contiguous
        )
        for (x_in, w_in, y) in outputs:
            want = expected
            if y is None:
                want = F.conv2d(x[:, :, :, 1:].float(), weight.float(), padding=padding)
                y = torch.full(want.shape, float("nan"), dtype=dtype, device="cuda")
            tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x_in, w_in, y)]
            assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, tag, *padding, 2, 0, 0) == 0
            assert runtime.last_launch().startswith("conv2d path 2"), runtime.last_launch()
            assert torch.allclose(y.float(), want, **HALF_TOL), (channels, r, s_, tuple(y.stride()), float((y.float() - want).abs().max()))
        untouched = torch.ones_like(wide, dtype=torch.bool)
        untouched[:, 2 : 2 + k, 1 : 1 + p, 3 : 3 + q] = False
        assert bool((wide[untouched] == 7).all())


def test_conv2d_one_launch_path_refuses_what_it_cannot_run():
    from ninetoothed_amd import runtime

    def call(n, c, h, w, k, r, s, padding):
        x = torch.zeros(n, c, h, w, dtype=torch.float16, device="cuda")
        weight = torch.zeros(k, c, r, s, dtype=torch.float16, device="cuda")
        out = torch.zeros(n, k, h + 2 * padding[0] - r + 1, w + 2 * padding[1] - s + 1, dtype=torch.float16, device="cuda")
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, out)]
        return runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, runtime.DATA_TYPE_INDEX["fp16"], padding[0], padding[1], 3, 0, 0)

    assert call(2, 32, 16, 16, 256, 7, 7, (3, 1)) == runtime.NO_KERNEL   # taps repeat only after 49 tiles
    assert call(2, 32, 16, 15, 256, 3, 3, (1, 1)) == runtime.NO_KERNEL   # output rows of 15 pixels
    assert call(2, 24, 16, 16, 256, 3, 3, (1, 1)) == runtime.NO_KERNEL   # C * R * S not a multiple of 32
    assert call(2, 32, 16, 16, 64, 3, 3, (1, 1)) == runtime.NO_KERNEL    # a quarter of a tile of output channels


def test_scratch_buffers_are_reused_grown_and_released():
    """conv2d's repacked operands and fp32 attention's narrowed K / V live in buffers the library
    keeps per stream: a smaller call after a larger one, a larger one after that, another stream and
    a call after nt_release_workspaces all have to give the same results."""
    from ninetoothed_amd import runtime

    def conv_case(n, c, hw, k):
        x, w = _randn(n, c, hw, hw, scale=0.1).cuda(), _randn(k, c, 3, 3, scale=0.1).cuda()
        return x, w, F.conv2d(x.float(), w.float(), padding=1).half()

    def repacked(x, w):  # the way that uses scratch memory, by name
        out = torch.full((x.shape[0], w.shape[0], x.shape[2], x.shape[3]), float("nan"), dtype=x.dtype, device="cuda")
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, w, out)]
        runtime.check(runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, runtime.DATA_TYPE_INDEX["fp16"], 1, 1, 2, 0, 0))
        return out

    cases = [conv_case(4, 64, 16, 256), conv_case(2, 32, 24, 256), conv_case(8, 64, 24, 512)]
    side = torch.cuda.Stream()
    for round_ in range(2):
        for x, w, expected in cases:
            assert torch.allclose(repacked(x, w), expected, **HALF_TOL)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            x, w, expected = cases[0]
            assert torch.allclose(repacked(x, w), expected, **HALF_TOL)
        side.synchronize()
        # (a head dimension without an fp32 kernel of its own: K and V are narrowed into the scratch buffer)
        q, k, v = (torch.randn(1, 2, 300 - 100 * round_, 96, device="cuda") for _ in range(3))
        o = _attention(q, k, v, scale=0.125)
        assert torch.allclose(o, F.scaled_dot_product_attention(q, k, v, scale=0.125), rtol=0.025, atol=0.025)
        torch.cuda.synchronize()
        runtime.library().nt_release_workspaces()


def test_first_launch_times_the_attention_variants_and_the_conv2d_paths():
    """Like a product with tunable block sizes, the first launch of a new attention / conv2d problem times the
    alternatives (loop variants; one launch on NCHW, repacking pass, gather kernel), records the winner, and
    later launches -- also of a kernel object made afterwards -- run it.  Every launch is checked."""
    from ninetoothed_amd import auto_tuner, runtime

    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    batch, heads, seq, dim = 3, 16, 640, 128  # sizes no other test uses (enough query blocks not to split the keys)
    q, k, v = (_randn(batch, heads, seq, dim).cuda() for _ in range(3))
    for is_causal in (False, True):
        problem = (fp16, batch, heads, seq, seq, dim, int(is_causal))
        assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, problem) < 0
        expected = _attention_reference(q, k, v, is_causal, dim**-0.5)
        for _ in range(2):  # the second kernel object starts from the recorded choice
            kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
            for _ in range(2):
                o = torch.full_like(q, float("nan"))
                kernel(q, k, v, is_causal, dim**-0.5, o)
                assert torch.allclose(o.float(), expected, **HALF_TOL)
            assert 0 <= auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, problem) <= 4
    # one query against a long key range splits the keys: nothing to choose from, nothing recorded
    q1 = _randn(1, 8, 1, 128).cuda()
    k1, v1 = _randn(1, 8, 8192, 128).cuda(), _randn(1, 8, 8192, 128).cuda()
    o1 = torch.full_like(q1, float("nan"))
    kernel(q1, k1, v1, False, dim**-0.5, o1)
    assert torch.allclose(o1.float(), _attention_reference(q1, k1, v1, False, dim**-0.5), **HALF_TOL)
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, (fp16, 1, 8, 1, 8192, 128, 0)) < 0

    n, c, h, w, kk = 3, 64, 24, 40, 256
    x, weight = _randn(n, c, h, w, scale=0.2).cuda(), _randn(kk, c, 3, 3, scale=0.2).cuda()
    problem = (fp16, n, c, h, w, kk, 3, 3, 1, 1, 1)
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, problem) < 0
    expected = F.conv2d(x.float(), weight.float(), padding=1)
    for _ in range(2):
        assert torch.allclose(_conv2d(x, weight, (1, 1)).float(), expected, **HALF_TOL)
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, problem) in (1, 2, 3)  # (4, the batched product, is for 1 x 1 filters)
    # each way by name (block_size_m of the C entry point), whole output
    for path in (1, 2, 3):
        y = torch.full((n, kk, h, w), float("nan"), dtype=torch.float16, device="cuda")
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
        assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 1, 1, path, 0, 0) == 0
        assert torch.allclose(y.float(), expected, **HALF_TOL), path


def test_a_tuned_pointwise_convolution_stays_on_the_batched_product():
    """1 x 1 filters without padding run as one batched launch of the GEMM kernels; the first-launch tuner has that
    way among its candidates (path 4, first in the order of preference), so a tuned problem does not end up on the
    repacking or gather kernel for the rest of the process.  ``nt_last_launch`` names what ran."""
    from ninetoothed_amd import auto_tuner, runtime

    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    n, c, h, w, kk = 5, 256, 24, 24, 64  # 64 output channels: the one-launch path (3) refuses it
    x, weight = _randn(n, c, h, w, scale=0.2).cuda(), _randn(kk, c, 1, 1, scale=0.2).cuda()
    problem = (fp16, n, c, h, w, kk, 1, 1, 0, 0, 1)
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, problem) < 0
    expected = F.conv2d(x.float(), weight.float())
    for _ in range(2):
        assert torch.allclose(_conv2d(x, weight, (0, 0)).float(), expected, **HALF_TOL)
        assert runtime.last_launch().startswith("conv2d path 4: "), runtime.last_launch()
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, problem) == 4
    # by name through the C ABI; a 3 x 3 filter is not that kind of problem
    y = torch.full((n, kk, h, w), float("nan"), dtype=torch.float16, device="cuda")
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 0, 0, 4, 0, 0) == 0
    assert torch.allclose(y.float(), expected, **HALF_TOL)
    weight3 = _randn(kk, c, 3, 3, scale=0.2).cuda()
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight3, y)]
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 1, 1, 4, 0, 0) == runtime.NO_KERNEL


def test_last_launch_names_the_kernel_that_ran_and_tuning_repeats_its_choice():
    """``nt_last_launch`` reports the instance / variant / path of the calling thread's latest launch, and timing the
    same problem again gives the same choice (interleaved rounds, per-candidate minima, a margin for the untuned
    rule's candidate)."""
    import ctypes

    from ninetoothed_amd import auto_tuner, runtime

    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    a, b = _randn(512, 512).cuda(), _randn(512, 512).cuda()
    c = torch.empty(512, 512, dtype=torch.float16, device="cuda")
    _matmul_kernel()(a, b, c)
    assert runtime.last_launch().startswith("gemm instance "), runtime.last_launch()
    x = torch.randn(64, 1000, device="cuda")
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    kernel(x, torch.empty_like(x), BLOCK_SIZE=1000)
    assert runtime.last_launch().startswith("softmax kernel "), runtime.last_launch()

    q, k, v = (_randn(2, 16, 1152, 128).cuda() for _ in range(3))
    o = torch.empty_like(q)
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (q, k, v, o)]
    choices = []
    for _ in range(3):
        best, best_ms = ctypes.c_int(-2), ctypes.c_float(0.0)
        causal, scale = runtime.ArgumentTensor.from_scalar(1), runtime.ArgumentTensor.from_scalar(128**-0.5)
        runtime.check(runtime.library().nt_tune_attention(runtime.current_stream(), tensors[0], tensors[1], tensors[2], causal, scale, tensors[3], fp16, 5, ctypes.byref(best), ctypes.byref(best_ms)))
        assert 0 <= best.value <= 4 and best_ms.value > 0.0
        choices.append(best.value)
    assert len(set(choices)) == 1, choices
    runtime.check(runtime.library().launch_nt_attention(runtime.current_stream(), tensors[0], tensors[1], tensors[2], causal, scale, tensors[3], fp16, 0, 0))
    assert runtime.last_launch().startswith(f"attention variant {choices[0]}: "), runtime.last_launch()
    assert torch.allclose(o.float(), _attention_reference(q, k, v, True, 128**-0.5), **HALF_TOL)
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, (fp16, 2, 16, 1152, 1152, 128, 1)) == choices[0]


def test_conv2d_one_launch_path_leaves_overlapping_images_to_the_other_ways():
    """The one-launch kernel assumes that offsets grow with (image, channel, row); an input whose images share
    memory (``expand`` over the batch: stride 0) is refused by it and runs correctly on another way."""
    from ninetoothed_amd import runtime

    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    x = _randn(1, 32, 16, 16, scale=0.3).cuda().expand(4, 32, 16, 16)
    weight = _randn(256, 32, 3, 3, scale=0.3).cuda()
    y = torch.full((4, 256, 16, 16), float("nan"), dtype=torch.float16, device="cuda")
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y)]
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 1, 1, 3, 0, 0) == runtime.NO_KERNEL
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 1, 1, 0, 0, 0) == 0
    assert torch.allclose(y.float(), F.conv2d(x.float(), weight.float(), padding=1), **HALF_TOL)
    # rows that overlap (a row stride shorter than a row) as well
    base = _randn(2, 32, 16 * 8 + 16, scale=0.3).cuda()
    x = base.as_strided((2, 32, 16, 16), (base.stride(0), base.stride(1), 8, 1))
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (x, weight, y[:2])]
    assert runtime.library().launch_nt_conv2d(runtime.current_stream(), *tensors, fp16, 1, 1, 3, 0, 0) == runtime.NO_KERNEL


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
def test_calls_that_run_on_copies_inside_a_captured_graph():
    """fp8 operands, operands the direct-to-LDS kernels cannot read in place and attention tensors with an odd head
    dimension run on copies in scratch buffers.  A capture that meets such a call before any eager call of its size
    cannot allocate: the products then take the kernels that need no scratch memory (an attention call of this kind
    has none and would be refused there), and after one eager call on the stream a capture of the same calls uses its
    buffers.
    Every replay is checked against the eager result, with eager work between the replays."""
    from ninetoothed_amd import runtime

    matmul = _matmul_kernel()
    attention = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(with_scale=True))
    m, n, k = 1544, 1160, 1208  # sizes no other test uses; 2^31 multiply-adds and more
    a8 = torch.randn(m, k, device="cuda").to(torch.float8_e5m2)
    b8 = torch.randn(k, n, device="cuda").to(torch.float8_e5m2)
    a_off = torch.randn(m, k + 1, dtype=torch.float16, device="cuda")[:, :k]  # rows off 16-byte boundaries
    b16 = torch.randn(k, n, dtype=torch.float16, device="cuda")
    q, kk, v = (torch.randn(2, 3, 150, 44, dtype=torch.float16, device="cuda") for _ in range(3))
    c8, c16 = torch.empty(m, n, dtype=torch.float16, device="cuda"), torch.empty(m, n, dtype=torch.float16, device="cuda")
    o = torch.empty_like(q)
    expected8 = a8.to(torch.float16).float() @ b8.to(torch.float16).float()
    expected16 = a_off.float() @ b16.float()
    expected_o = _attention_reference(q, kk, v, False, 44**-0.5)
    tolerance = dict(rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)

    def products():
        matmul(a8, b8, c8)
        matmul(a_off, b16, c16)

    def replay_and_check(graph, with_attention):
        for replay in range(3):
            for t in (c8, c16, o):
                t.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.allclose(c8.float(), expected8, **tolerance), replay
            assert torch.allclose(c16.float(), expected16, **tolerance), replay
            if with_attention:
                assert torch.allclose(o.float(), expected_o, **HALF_TOL), replay
            (a_off.float() @ b16.float()).sum().item()  # eager work between the replays

    runtime.library().nt_release_workspaces()  # no buffer of any size exists
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    first = torch.cuda.CUDAGraph()
    with torch.cuda.graph(first, stream=stream):
        products()
        assert "any-stride" in runtime.last_launch(), runtime.last_launch()  # no scratch memory: the kernel that gathers in place
    replay_and_check(first, with_attention=False)
    # eager calls on that stream allocate its buffers (they are kept per stream) ...
    with torch.cuda.stream(stream):
        products()
        assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
        attention(q, kk, v, False, 44**-0.5, o)
    torch.cuda.synchronize()
    assert torch.allclose(o.float(), expected_o, **HALF_TOL)
    # ... and a capture of the same calls then runs on the copies
    second = torch.cuda.CUDAGraph()
    with torch.cuda.graph(second, stream=stream):
        products()
        assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
        attention(q, kk, v, False, 44**-0.5, o)
    replay_and_check(second, with_attention=True)


def test_first_call_of_an_untuned_problem_inside_a_captured_graph():
    """Nothing has run these problems before the capture starts: the first-launch tuner of the product
    (event synchronisation, repeated launches) and the specialisation of the tile map (compiling and
    loading code) would both break a capture.  Inside one the product takes the untuned choice and the
    tile map its interpreter kernel; the first call outside a capture then tunes / specialises."""
    from ninetoothed_amd import auto_tuner, runtime

    m, n, k = 264, 520, 776  # sizes no other test uses
    a, b, bias = _randn(m, k).cuda(), _randn(k, n, scale=0.1).cuda(), _randn(m, n).cuda()
    c, d = torch.empty(m, n, dtype=torch.float16, device="cuda"), torch.empty(m, n, dtype=torch.float16, device="cuda")
    x, y = torch.randn(1237, device="cuda"), torch.randn(1237, device="cuda")
    z = torch.empty_like(x)
    matmul = _matmul_kernel()
    addmm = ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())

    def arrangement(lhs, rhs, output, block=ninetoothed.block_size()):
        return lhs.tile((block,)), rhs.tile((block,)), output.tile((block,))

    def application(lhs, rhs, output):
        output = lhs * 3.25 + rhs * rhs - 0.0078125  # noqa: F841

    tile_map = ninetoothed.make(arrangement, application, (Tensor(1),) * 3)
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    assert auto_tuner.enabled() and auto_tuner.lookup(fp16, fp16, m, n, k, False) < 0 and auto_tuner.lookup(fp16, fp16, m, n, k, True) < 0

    qa, ka, va = (_randn(2, 3, 328, 64).cuda() for _ in range(3))
    oa = torch.empty_like(qa)
    xc, wc = _randn(2, 32, 16, 24, scale=0.2).cuda(), _randn(256, 32, 3, 3, scale=0.2).cuda()
    yc = torch.empty(2, 256, 16, 24, dtype=torch.float16, device="cuda")
    attention = ninetoothed.make(programs.attention.arrangement, programs.attention.application, programs.attention.tensors())
    conv = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    attention_problem = (fp16, 2, 3, 328, 328, 64, 1)
    conv_problem = (fp16, 2, 32, 16, 24, 256, 3, 3, 1, 1, 1)

    def run():
        matmul(a, b, c)
        addmm(bias, a, b, 0.5, 2.0, d)
        tile_map(x, y, z)
        attention(qa, ka, va, True, oa)
        conv(xc, wc, yc, padding_h=1, padding_w=1)

    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        run()
    assert auto_tuner.lookup(fp16, fp16, m, n, k, False) < 0  # nothing was timed during the capture
    assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, attention_problem) < 0
    assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, conv_problem) < 0
    product = a.float() @ b.float()
    expected = (product, 0.5 * bias.float() + 2.0 * product.half().float(), x * 3.25 + y * y - 0.0078125)
    expected_attention = _attention_reference(qa, ka, va, True, 1.4423828125 / 1.4426950408889634)  # (the program's literal, rounded to fp16)
    expected_conv = F.conv2d(xc.float(), wc.float(), padding=1)
    for replay in range(3):
        for t in (c, d, z, oa, yc):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.allclose(c.float(), expected[0], **HALF_TOL), replay
        assert torch.allclose(d.float(), expected[1], rtol=1e-2, atol=2e-2), replay
        assert torch.allclose(z, expected[2], rtol=1e-6, atol=1e-6), replay
        assert torch.allclose(oa.float(), expected_attention, **HALF_TOL), replay
        assert torch.allclose(yc.float(), expected_conv, **HALF_TOL), replay
        if replay == 0:
            run()  # the first eager call tunes the products, attention and the convolution and specialises the tile map
            torch.cuda.synchronize()
            assert auto_tuner.lookup(fp16, fp16, m, n, k, False) >= 0 and auto_tuner.lookup(fp16, fp16, m, n, k, True) >= 0
            assert auto_tuner.lookup_problem(runtime.TUNE_ATTENTION, attention_problem) >= 0
            assert auto_tuner.lookup_problem(runtime.TUNE_CONV2D, conv_problem) >= 1
            assert torch.allclose(z, expected[2], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("warm_on_capture_stream", (False, True))
def test_calls_that_use_scratch_memory_inside_a_captured_graph(warm_on_capture_stream):
    """A split-K product, a decoding attention and a convolution captured into a HIP graph.  Warmed
    up on the capture stream, the stream's scratch buffers exist and the captured kernels reuse them
    on every replay; warmed up elsewhere, nothing may be allocated during capture and the calls take
    their scratch-free kernels.  Replayed three times with eager work in between, each replay
    checked against the eager results."""
    a, b = _randn(16, 4096).cuda(), _randn(4096, 1024, scale=0.1).cuda()
    q, k, v = _randn(1, 4, 1, 64).cuda(), _randn(1, 4, 4096, 64).cuda(), _randn(1, 4, 4096, 64).cuda()
    x, w = _randn(2, 64, 16, 16, scale=0.1).cuda(), _randn(64, 64, 3, 3, scale=0.1).cuda()
    c = torch.empty(16, 1024, dtype=torch.float16, device="cuda")
    o = torch.empty_like(q)
    y = torch.empty(2, 64, 16, 16, dtype=torch.float16, device="cuda")
    matmul = _matmul_kernel()
    attention = ninetoothed.make(programs.attention.arrangement, programs.attention.application, programs.attention.tensors())
    conv = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())

    def run():
        matmul(a, b, c)
        attention(q, k, v, False, o)
        conv(x, w, y, padding_h=1, padding_w=1)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream if warm_on_capture_stream else torch.cuda.current_stream()):
        run()  # also lets the first-launch tuner (which synchronises) finish outside the capture
    torch.cuda.synchronize()
    expected = (a.float() @ b.float(), _attention_reference(q, k, v, False, 1.0), F.conv2d(x.float(), w.float(), padding=1))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        run()
    for replay in range(3):
        for t in (c, o, y):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.allclose(c.float(), expected[0], **HALF_TOL), replay
        assert torch.allclose(o.float(), expected[1], **HALF_TOL), replay
        assert torch.allclose(y.float(), expected[2], **HALF_TOL), replay
        run()  # eager work between the replays
        torch.cuda.synchronize()


# ---- tile selection -------------------------------------------------------------


def test_first_launch_tunes_and_the_choice_persists(tmp_path, monkeypatch):
    import ctypes

    from ninetoothed_amd import auto_tuner, runtime

    monkeypatch.setattr(auto_tuner, "CACHE_DIR", tmp_path)
    lib = runtime.library()
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    # a problem this process has not tuned yet (the table is per process and other tests launch products too)
    m, n, k = next(shape for shape in ((768, 1280, 512), (1280, 768, 512), (768, 1536, 512), (1792, 768, 512)) if lib.nt_tune_cache_lookup(fp16, fp16, *shape, 0) == -1)
    a, b = _randn(m, k).cuda(), _randn(k, n).cuda()
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application_with_cast, programs.matmul.tensors())
    kernel(a, b, out)
    assert torch.allclose(out, torch.matmul(a, b), **HALF_TOL)
    choice = lib.nt_tune_cache_lookup(fp16, fp16, m, n, k, 0)
    assert 0 <= choice < lib.nt_gemm_num_configs()
    files = list(tmp_path.glob("gemm_*.csv"))
    assert len(files) == 1
    entries = ctypes.c_int(0)
    assert lib.nt_tune_cache_load(str(files[0]).encode(), ctypes.byref(entries)) == 0 and entries.value >= 1
    # every instance that accepts the problem gives the same answer as the tuned launch
    null = runtime.ArgumentTensor.null()
    for config in range(lib.nt_gemm_num_configs()):
        other = torch.full_like(out, float("nan"))
        code = lib.launch_nt_gemm_config(
            runtime.current_stream(), config, null, runtime.ArgumentTensor.from_torch_tensor(a), runtime.ArgumentTensor.from_torch_tensor(b),
            null, null, runtime.ArgumentTensor.from_torch_tensor(other), fp16, fp16,
        )
        assert code in (0, runtime.NO_KERNEL)
        if code == 0:
            assert torch.allclose(other, out, **HALF_TOL)


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
@pytest.mark.parametrize("m, n, k", ((512, 512, 512), (130, 70, 45)))
def test_matmul_float8_e5m2_operands(m, n, k):
    # tests/test_matmul.py:61-88 of the reference: fp8 operands (the right one column-major), fp16 output,
    # compared with the fp16 product of the widened operands at atol 0.125; widening is exact, so the
    # oracle on the widened operands must agree to fp16 rounding as well
    lhs = _randn(m, k).to(torch.float8_e5m2)
    rhs = _randn(n, k).to(torch.float8_e5m2).T  # shape (k, n), strides (1, k)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
    kernel(lhs.cuda(), rhs.cuda(), out)
    _native_only(kernel, "launch_nt_matmul")
    expected = torch.matmul(lhs.to(torch.float16).cuda(), rhs.to(torch.float16).cuda())
    assert torch.allclose(out, expected, atol=0.125)
    reference = oracle.matmul(lhs.to(torch.float16).numpy(), np.ascontiguousarray(rhs.to(torch.float16).numpy()), bm=64, bn=64, bk=64)
    assert np.allclose(out.cpu().float().numpy(), reference, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_large_products_on_operands_the_fast_instances_cannot_read_run_on_dense_copies(dtype):
    """A K that is no multiple of 8, rows off 16-byte boundaries, an lhs stored by columns, other strides: from 2^21
    multiply-adds on such operands are copied (k contiguous, K padded to 8 with zeros) and the product runs on the
    direct-to-LDS instances; an output stored by columns runs as the transposed product.  What lies next to the operands in memory is Inf and must not reach the sums; what
    lies next to the output must stay as it was."""
    from ninetoothed_amd import runtime

    kernel = _matmul_kernel()

    def inside(rows, cols, pad_rows=1, pad_cols=3, transposed=False):
        # a [rows, cols] matrix inside an Inf-filled buffer; `transposed`: stored by columns
        shape = (cols + pad_rows, rows + pad_cols) if transposed else (rows + pad_rows, cols + pad_cols)
        buffer = torch.full(shape, float("inf"), dtype=dtype, device="cuda")
        view = buffer[: shape[0] - pad_rows, : shape[1] - pad_cols]
        view.copy_(torch.randn(view.shape, device="cuda").to(dtype))
        return view.T if transposed else view

    def check(lhs, rhs, out_cols_pad=0, fast=True):
        m, k, n = lhs.shape[0], lhs.shape[1], rhs.shape[1]
        buffer = torch.full((m + 1, n + out_cols_pad + 8), 7.0, dtype=dtype, device="cuda")
        out = buffer[:m, :n]
        kernel(lhs, rhs, out)
        _native_only(kernel, "launch_nt_matmul")
        assert ("any-stride" not in runtime.last_launch()) == fast, runtime.last_launch()
        expected = lhs.float() @ rhs.float()
        assert torch.allclose(out.float(), expected, rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5), float((out.float() - expected).abs().max())
        assert bool((buffer[m:] == 7.0).all()) and bool((buffer[:, n:] == 7.0).all())

    check(inside(2050, 1029), inside(1029, 1100))                      # K = 1029, rows off 16-byte boundaries, N no multiple of 8
    check(inside(2048, 1024, transposed=True), inside(1024, 1024))     # the lhs stored by columns
    check(inside(2048, 1024, transposed=True), inside(1024, 1031, transposed=True), out_cols_pad=1)  # both, C rows off 16-byte boundaries
    wide_l, wide_r = inside(2048, 2048), inside(1024, 2048)
    check(wide_l[:, ::2], wide_r[:, ::2])                              # every other column
    # an output stored by columns: the transposed product, here on dense operands and on ones that need copies
    for lhs, rhs in ((torch.randn(1024, 512, device="cuda").to(dtype), torch.randn(512, 768, device="cuda").to(dtype)), (inside(1030, 517), inside(517, 771))):
        buffer = torch.full((rhs.shape[1] + 1, lhs.shape[0] + 8), 7.0, dtype=dtype, device="cuda")
        out = buffer[: rhs.shape[1], : lhs.shape[0]].T
        kernel(lhs, rhs, out)
        assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
        assert torch.allclose(out.float(), lhs.float() @ rhs.float(), **HALF_TOL)
        assert bool((buffer[rhs.shape[1] :] == 7.0).all()) and bool((buffer[:, lhs.shape[0] :] == 7.0).all())
    # small products as well (the any-stride kernel is slower from 128^3 on) ...
    check(inside(300, 205), inside(205, 301))
    # ... and below that it serves the call as before
    check(inside(100, 77), inside(77, 90), fast=False)
    # addmm on such operands, the bias with rows off 16-byte boundaries as well
    m, k, n = 2050, 1029, 1100
    bias, lhs, rhs = inside(m, n), inside(m, k), inside(k, n)
    buffer = torch.full((m + 1, n + 9), 7.0, dtype=dtype, device="cuda")
    out = buffer[:m, :n]
    application = programs.addmm.application if dtype == torch.float16 else programs.addmm.application_bfloat16
    addmm = ninetoothed.make(programs.addmm.arrangement, application, programs.addmm.tensors())
    addmm(bias, lhs, rhs, 0.5, 2.0, out)
    _native_only(addmm, "launch_nt_addmm")
    assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
    expected = 0.5 * bias.float() + 2.0 * (lhs.float() @ rhs.float()).to(dtype).float()
    tolerance = dict(rtol=2e-2, atol=2e-2 * (k / 512) ** 0.5) if dtype == torch.bfloat16 else dict(rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)
    assert torch.allclose(out.float(), expected, **tolerance), float((out.float() - expected).abs().max())
    assert bool((buffer[m:] == 7.0).all()) and bool((buffer[:, n:] == 7.0).all())


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
def test_matmul_float8_e5m2_large_products_run_on_widened_copies():
    """fp8 operands are widened into fp16 copies (exact) and the product runs on the fp16 instances, direct-to-LDS
    where the copies allow: every layout the copies have to follow, against the fp32 product of the widened operands
    and against the widening any-stride kernel named through the C ABI."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    fp8, fp16, fp32 = (runtime.DATA_TYPE_INDEX[name] for name in ("fp8e5m2", "fp16", "fp32"))
    null = runtime.ArgumentTensor.null()
    kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())

    def check(lhs, rhs, out_dtype=torch.float16, fast=True):
        m, n = lhs.shape[0], rhs.shape[1]
        out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        kernel(lhs, rhs, out)
        _native_only(kernel, "launch_nt_matmul")
        assert ("any-stride" not in runtime.last_launch()) == fast, runtime.last_launch()
        product = lhs.to(torch.float16).float() @ rhs.to(torch.float16).float()
        k = lhs.shape[1]
        assert torch.allclose(out.float(), product, rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)
        plain = torch.full_like(out, float("nan"))
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (lhs, rhs, plain)]
        assert lib.launch_nt_gemm_config(runtime.current_stream(), 0, null, tensors[0], tensors[1], null, null, tensors[2], fp8, fp32 if out_dtype == torch.float32 else fp16) == 0
        assert torch.allclose(out.float(), plain.float(), rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)

    m, n, k = 2048, 1024, 1024
    lhs = torch.randn(m, k, device="cuda").to(torch.float8_e5m2)
    rhs = torch.randn(k, n, device="cuda").to(torch.float8_e5m2)
    check(lhs, rhs)                                      # both row-major
    check(lhs, rhs, out_dtype=torch.float32)
    check(lhs, torch.randn(n, k, device="cuda").to(torch.float8_e5m2).T)   # the reference's case: the rhs column-major
    check(torch.randn(k, m, device="cuda").to(torch.float8_e5m2).T, rhs)  # a column-major lhs: the widened copy follows it and is copied once more, k contiguous
    # operands inside wider buffers, rows that start off 16-byte boundaries (byte-wise widening)
    wide = torch.randn(m + 3, k + 5, device="cuda").to(torch.float8_e5m2)
    lhs2 = wide[3:, 5:]
    lhs2.view(torch.uint8)[0, 0] = 0x5C  # 256.0
    check(lhs2, rhs)
    # sizes that are no multiples of 8: the widened copies get padded rows and are copied once more, K padded to 8
    check(torch.randn(2050, 1030, device="cuda").to(torch.float8_e5m2), torch.randn(1030, 1001, device="cuda").to(torch.float8_e5m2))
    # addmm: the bias is widened as well (tests/test_addmm.py:57-90 of the reference at a larger size)
    bias = torch.randn(m, n, device="cuda").to(torch.float8_e5m2)
    rhs_t = torch.randn(n, k, device="cuda").to(torch.float8_e5m2).T
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    addmm = ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())
    addmm(bias, lhs, rhs_t, 0.37, 0.81, out)
    _native_only(addmm, "launch_nt_addmm")
    assert "any-stride" not in runtime.last_launch(), runtime.last_launch()
    product = (lhs.to(torch.float16).float() @ rhs_t.to(torch.float16).float()).half().float()
    assert torch.allclose(out.float(), 0.37 * bias.to(torch.float16).float() + 0.81 * product, rtol=1e-2, atol=2e-2 * (k / 512) ** 0.5)


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
def test_addmm_float8_e5m2_operands():
    # tests/test_addmm.py:57-90 of the reference: fp8 input, mat1, mat2 (the last column-major), fp16 output
    m, n, k = 512, 512, 512
    input = _randn(m, n).to(torch.float8_e5m2)
    mat1 = _randn(m, k).to(torch.float8_e5m2)
    mat2 = _randn(n, k).to(torch.float8_e5m2).T
    beta, alpha = 0.37, 0.81
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel = ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())
    kernel(input.cuda(), mat1.cuda(), mat2.cuda(), beta, alpha, out)
    _native_only(kernel, "launch_nt_addmm")
    widened = [t.to(torch.float16) for t in (input, mat1, mat2)]
    expected = torch.addmm(widened[0].cuda(), widened[1].cuda(), widened[2].cuda(), beta=beta, alpha=alpha)
    assert torch.allclose(out, expected, atol=0.075)
    reference = oracle.addmm(widened[0].numpy(), widened[1].numpy(), np.ascontiguousarray(widened[2].numpy()), beta, alpha)
    assert np.allclose(out.cpu().float().numpy(), reference, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16, torch.float32))
@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_tensors_the_kernels_cannot_read_in_place_run_on_padded_copies(is_causal, dtype):
    """Head dimensions that are no multiples of 8 (the reference pads them to a power of two and masks:
    src/ninetoothed/generation.py:563-574), rows off 16-byte boundaries, a strided last dimension: Q, K and V are
    copied into padded dense buffers, O is copied back.  The tensors lie inside Inf-filled buffers (nothing next to
    them may reach the sums) and O inside sentinels."""
    tolerance = dict(rtol=1e-3, atol=1e-3) if dtype == torch.float32 else HALF_TOL
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(with_scale=True))

    def inside(b, h, s, d, pad=3, step=1):
        buffer = torch.full((b, h, s + 1, d * step + pad), float("inf"), dtype=dtype, device="cuda")
        view = buffer[:, :, :s, 1 : 1 + d * step : step]
        view.copy_(torch.randn(b, h, s, d, device="cuda").to(dtype))
        return view

    for (b, h, sq, sk, d, step) in ((2, 3, 200, 200, 100, 1), (1, 4, 130, 77, 20, 1), (2, 2, 64, 300, 12, 1), (1, 2, 257, 257, 64, 1), (1, 2, 100, 100, 36, 2), (1, 1, 50, 50, 250, 1)):
        if is_causal and sq != sk:
            continue
        q, k, v = inside(b, h, sq, d, step=step), inside(b, h, sk, d, step=step), inside(b, h, sk, d, step=step)
        buffer = torch.full((b, h, sq + 1, d + 5), 7.0, dtype=dtype, device="cuda")
        o = buffer[:, :, :sq, 2 : 2 + d]
        kernel(q, k, v, is_causal, d**-0.5, o)
        _native_only(kernel, "launch_nt_attention")
        expected = _attention_reference(q, k, v, is_causal, d**-0.5)
        assert torch.allclose(o.float(), expected, **tolerance), (b, h, sq, sk, d, float((o.float() - expected).abs().max()))
        assert bool((buffer[:, :, sq:] == 7.0).all()) and bool((buffer[:, :, :, :2] == 7.0).all()) and bool((buffer[:, :, :, 2 + d :] == 7.0).all())


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("seq_len", (1024, 1))
def test_attention_float32_tensors(seq_len, is_causal):
    # the fp32 case of tests/test_attention.py:99-117 of the reference, with its tolerance
    q, k, v = (torch.randn(2, 4, seq_len, 64, generator=torch.Generator().manual_seed(s)) for s in (0, 1, 2))
    out = _attention(q.cuda(), k.cuda(), v.cuda(), is_causal)
    expected = F.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=is_causal, scale=1)
    assert out.dtype == torch.float32
    assert torch.allclose(out, expected, rtol=0.025, atol=0.025)
    # strided K / V (a transposed view) go through the same conversion
    k_view = k.transpose(1, 2).contiguous().transpose(1, 2)
    assert torch.allclose(_attention(q.cuda(), k_view.cuda(), v.cuda(), is_causal), expected, rtol=0.025, atol=0.025)


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("batch, heads, seq_q, seq_k, emb_dim", ((2, 3, 200, 200, 64), (1, 2, 77, 77, 128), (2, 2, 130, 130, 32), (1, 3, 50, 211, 64), (1, 2, 300, 45, 128)))
@pytest.mark.parametrize("pad", (4, 3))
def test_attention_float32_tensors_are_not_narrowed(batch, heads, seq_q, seq_k, emb_dim, is_causal, pad):
    """Head dimensions 32, 64 and 128 of fp32 tensors run in fp32 throughout: against a float64 reference at fp32
    tolerances, on operands that the fp16 range does not hold (keys around 1e5 against queries around 1e-5, values
    around 1e6), ragged and unequal lengths, K and V inside Inf-filled rows -- whose pitch is a multiple of 16 bytes
    or not: the precision of the result must not depend on where the rows of K start."""
    generator = torch.Generator().manual_seed(seq_q + emb_dim)
    q = torch.randn(batch, heads, seq_q, emb_dim, generator=generator) * 1e-5
    wide_k = torch.full((batch, heads, seq_k, emb_dim + pad), float("inf"))
    wide_v = torch.full((batch, heads, seq_k, emb_dim + pad), float("inf"))
    wide_k[..., pad - 3 : pad - 3 + emb_dim] = torch.randn(batch, heads, seq_k, emb_dim, generator=generator) * 1e5
    wide_v[..., :emb_dim] = torch.randn(batch, heads, seq_k, emb_dim, generator=generator) * 1e6
    k, v = wide_k.cuda()[..., pad - 3 : pad - 3 + emb_dim], wide_v.cuda()[..., :emb_dim]
    scale = emb_dim**-0.5
    out = _attention(q.cuda(), k, v, is_causal, scale)
    assert out.dtype == torch.float32
    scores = (q.double().cuda() * scale) @ k.double().transpose(-1, -2)
    assert float(scores.abs().max()) > 2.0  # (the softmax is not flat)
    if is_causal:
        visible = torch.ones(seq_q, seq_k, dtype=torch.bool, device="cuda").tril()
        scores = scores.masked_fill(~visible, float("-inf"))
    expected = torch.softmax(scores, dim=-1) @ v.double()
    assert torch.allclose(out.double(), expected, rtol=2e-4, atol=2e-4 * 1e6)


def test_attention_float32_with_block_size_hints_runs_on_narrowed_copies():
    from ninetoothed_amd import runtime

    q, k, v = (torch.randn(2, 2, 150, 64, device="cuda") for _ in range(3))
    o = torch.full_like(q, float("nan"))
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (q, k, v)]
    causal, scale = runtime.ArgumentTensor.from_scalar(0), runtime.ArgumentTensor.from_scalar(0.125)
    fp32 = runtime.DATA_TYPE_INDEX["fp32"]
    runtime.check(runtime.library().launch_nt_attention(runtime.current_stream(), *tensors, causal, scale, runtime.ArgumentTensor.from_torch_tensor(o), fp32, 128, 64))
    assert torch.allclose(o, F.scaled_dot_product_attention(q, k, v, scale=0.125), rtol=0.025, atol=0.025)


@pytest.mark.parametrize("m", (1, 100, 1000, 4097))
@pytest.mark.parametrize("addmm", (False, True))
def test_gemm_any_number_of_rows_on_the_direct_to_lds_path(m, addmm):
    # M need not be a multiple of the tile: rows past the end read as zeros and are not stored
    from ninetoothed_amd import runtime

    n, k = 1024, 512
    a, b = _randn(m, k).cuda(), _randn(k, n, scale=0.1).cuda()
    guard = torch.full((m + 64, n), 7.0, dtype=torch.float16, device="cuda")  # rows after the output must stay untouched
    out = guard[:m]
    lib = runtime.library()
    names = runtime.gemm_config_names()
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    null = runtime.ArgumentTensor.null()
    if addmm:
        input = _randn(m, n).cuda()
        expected = torch.addmm(input, a, b, beta=0.5, alpha=2.0)
        extra = (runtime.ArgumentTensor.from_torch_tensor(input), runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0))
    else:
        expected = torch.matmul(a, b)
        extra = (null, null, null)
    ran = 0
    for config, name in enumerate(names):
        if "lds-direct" not in name:
            continue
        out.fill_(float("nan"))
        code = lib.launch_nt_gemm_config(
            runtime.current_stream(), config, extra[0], runtime.ArgumentTensor.from_torch_tensor(a), runtime.ArgumentTensor.from_torch_tensor(b),
            extra[1], extra[2], runtime.ArgumentTensor.from_torch_tensor(out), fp16, fp16,
        )
        if code == 1 and "split-k" in name:  # only takes problems with few output tiles
            continue
        assert code == 0, name
        assert torch.allclose(out, expected, rtol=2e-2, atol=2e-2), name
        assert bool((guard[m:] == 7.0).all()), name
        ran += 1
    assert ran >= 4


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_gemm_large_tile_every_k_tile_count(dtype):
    """The 256x256x32 instance stages its lhs two k tiles at a time in a ring of three, its rhs one at a time in a
    ring of four, over a loop body of twelve steps: every number of k tiles from 1 to 27 (all residues of the body,
    odd counts leave half a pair unused), a partial tile of rows, through the C ABI by instance.  The lhs is a view
    into a wider matrix whose other columns hold Inf: reading past the k range of a row would show."""
    import ctypes

    from ninetoothed_amd import runtime

    lib = runtime.library()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    buffer = ctypes.create_string_buffer(128)
    instance = None
    for index in range(lib.nt_gemm_num_configs()):
        runtime.check(lib.nt_gemm_config_name(index, buffer, len(buffer)))
        if buffer.value.decode().startswith("256x256x32 waves 2x4 stages 5") and "tails" not in buffer.value.decode():
            instance = index
            break
    assert instance is not None
    null = runtime.ArgumentTensor.null()
    m, n = 300, 512
    for tiles in list(range(1, 28)) + [61]:
        k = 32 * tiles
        wide = torch.full((m, k + 64), float("inf"), dtype=dtype, device="cuda")
        wide[:, :k] = _randn(m, k, dtype=dtype).cuda()
        a = wide[:, :k]
        b = _randn(k, n, dtype=dtype).cuda()
        bias = _randn(m, n, dtype=dtype).cuda()
        out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        code = lib.launch_nt_gemm_config(
            runtime.current_stream(), instance, runtime.ArgumentTensor.from_torch_tensor(bias), runtime.ArgumentTensor.from_torch_tensor(a),
            runtime.ArgumentTensor.from_torch_tensor(b), runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0),
            runtime.ArgumentTensor.from_torch_tensor(out), tag, tag,
        )
        assert code == 0, (tiles, code)
        product = (a.float() @ b.float()).to(dtype).float()
        expected = 0.5 * bias.float() + 2.0 * product
        tolerance = dict(rtol=2e-2, atol=2e-2) if dtype == torch.float16 else dict(rtol=5e-2, atol=2e-1)
        assert torch.allclose(out.float(), expected, **tolerance), (tiles, float((out.float() - expected).abs().max()))


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((300, 200, 104), (1000, 1000, 1000), (257, 264, 72), (512, 520, 8), (2100, 3000, 2056)))
def test_gemm_partial_tiles_along_n_and_k(m, n, k, dtype):
    """N and K that do not fit the tile (multiples of 8) stay on the direct-to-LDS kernels: the
    instances with tails, row-major and transposed rhs, element-type / fp32 / addmm epilogues.
    Whole output, NaN-poisoned, inside a wider buffer whose extra columns must stay untouched.
    What lies next to the operands in memory is Inf: the element after a row's end (the next
    row's first), rows of the rhs past K -- none of it may reach the result."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    names = runtime.gemm_config_names()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    null = runtime.ArgumentTensor.null()
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0)
    # (plain products: rtol = atol = 1e-2 against the fp32 product; with a bias the product is rounded before it is
    # scaled by alpha = 2 and may be cancelled by the bias, so one ulp of the product sets the absolute tolerance)
    biased = dict(rtol=2e-2, atol=2e-2 * max(k / 512, 1) ** 0.5) if dtype == torch.bfloat16 else dict(rtol=1e-2, atol=1e-2 * max(k / 512, 1) ** 0.5)
    a = torch.randn(m, k, dtype=dtype, device="cuda")
    a[1, 0] = float("inf")  # follows row 0 in memory: only row 1 of the result may see it
    tall = torch.randn(k + 8, n, dtype=dtype, device="cuda")
    tall[k:] = float("inf")
    wide = torch.randn(n, k, dtype=dtype, device="cuda")
    wide[1, 0] = float("inf")  # transposed rhs: follows column 0's k range, belongs to column 1
    bias = torch.randn(m, n, dtype=dtype, device="cuda")
    for b, clean_rows, clean_cols in ((tall[:k], [r for r in range(m) if r != 1], slice(None)), (wide.t(), [r for r in range(m) if r != 1], [c for c in range(n) if c != 1])):
        product = (a.float() @ b.float())[clean_rows][:, clean_cols]
        assert bool(torch.isfinite(product).all())
        for out_dtype, with_bias in ((dtype, False), (torch.float32, False), (dtype, True)):
            buffer = torch.full((m, n + 24), 7.0, dtype=out_dtype, device="cuda")
            out = buffer[:, :n]
            tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
            expected = 0.5 * bias.float()[clean_rows][:, clean_cols] + 2.0 * product.to(dtype).float() if with_bias else product
            out_tag = runtime.DATA_TYPE_INDEX["fp32"] if out_dtype == torch.float32 else tag
            served = 0
            for instance, name in enumerate(names):
                if "tails" not in name or "split-k" in name:
                    continue
                out.fill_(float("nan"))
                result = lib.launch_nt_gemm_config(
                    runtime.current_stream(), instance, tensors[0] if with_bias else null, tensors[1], tensors[2], beta if with_bias else null,
                    alpha if with_bias else null, tensors[3], tag, out_tag,
                )
                assert result == 0, name
                served += 1
                assert torch.allclose(out.float()[clean_rows][:, clean_cols], expected, **(biased if with_bias else HALF_TOL)), (name, out_dtype, with_bias)
                assert bool((buffer[:, n:] == 7.0).all()), name
            assert served >= 3
        # through `make`: the heuristic picks an instance with tails instead of the any-stride kernel
        out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        _matmul_kernel()(a, b, out)
        assert torch.allclose(out.float()[clean_rows][:, clean_cols], product, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((300, 1001, 512), (64, 50257, 256), (1000, 77, 1032), (5, 3, 8)))
def test_gemm_transposed_rhs_any_number_of_columns(m, n, k, dtype):
    """`x @ w.T` with any number of rows of `w` (an odd vocabulary size): the operands still stream
    through LDS in 16-byte pieces, C -- whose rows are then not 16-byte aligned -- is stored
    element by element.  Every instance with tails, element-type / fp32 / addmm (any-stride input)."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    names = runtime.gemm_config_names()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    null = runtime.ArgumentTensor.null()
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0)
    # (plain products: rtol = atol = 1e-2 against the fp32 product; with a bias the product is rounded before it is
    # scaled by alpha = 2 and may be cancelled by the bias, so one ulp of the product sets the absolute tolerance)
    biased = dict(rtol=2e-2, atol=2e-2 * max(k / 512, 1) ** 0.5) if dtype == torch.bfloat16 else dict(rtol=1e-2, atol=1e-2 * max(k / 512, 1) ** 0.5)
    a = torch.randn(m, k, dtype=dtype, device="cuda")
    w = torch.randn(n, k, dtype=dtype, device="cuda")
    b = w.t()
    bias = torch.randn(m, n, dtype=dtype, device="cuda")
    product = a.float() @ b.float()
    for out_dtype, with_bias in ((dtype, False), (torch.float32, False), (dtype, True)):
        buffer = torch.full((m * n + 16,), 7.0, dtype=out_dtype, device="cuda")
        out = buffer[: m * n].view(m, n)
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
        expected = 0.5 * bias.float() + 2.0 * product.to(dtype).float() if with_bias else product
        out_tag = runtime.DATA_TYPE_INDEX["fp32"] if out_dtype == torch.float32 else tag
        served = 0
        for instance, name in enumerate(names):
            if "tails" not in name or "split-k" in name:
                continue
            out.fill_(float("nan"))
            result = lib.launch_nt_gemm_config(
                runtime.current_stream(), instance, tensors[0] if with_bias else null, tensors[1], tensors[2], beta if with_bias else null,
                alpha if with_bias else null, tensors[3], tag, out_tag,
            )
            assert result == 0, name
            served += 1
            assert torch.allclose(out.float(), expected, **(biased if with_bias else HALF_TOL)), (name, out_dtype, with_bias)
            assert bool((buffer[m * n :] == 7.0).all()), name
        assert served >= 3
    out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    _matmul_kernel()(a, b, out)
    assert torch.allclose(out.float(), product, **HALF_TOL)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("m, n, k", ((1, 2048, 4096), (16, 1024, 8192), (64, 520, 2056), (300, 200, 4104), (512, 512, 16384), (129, 136, 256), (768, 1032, 4096),
                                     (33, 515, 8192), (16, 1001, 4096), (100, 301, 5000), (7, 50, 2048)))
def test_gemm_split_k(m, n, k, dtype):
    """Few output tiles, long K: the k range is cut into parts that run as workgroups of their own
    and a second kernel sums them (fp32) and applies the epilogue.  Both rhs layouts, element-type /
    fp32 / addmm outputs, NaN-poisoned output with sentinel columns beside it; twice in a row
    (the scratch tensor of the stream is reused).  An N that is no multiple of 8 goes with a k-contiguous
    rhs (as in the one-pass instances): the partial tiles then have rows of N rounded up to 8 and the
    second kernel stores element by element."""
    from ninetoothed_amd import runtime

    lib = runtime.library()
    names = runtime.gemm_config_names()
    tag = runtime.DATA_TYPE_INDEX["fp16" if dtype == torch.float16 else "bf16"]
    null = runtime.ArgumentTensor.null()
    beta, alpha = runtime.ArgumentTensor.from_scalar(0.5), runtime.ArgumentTensor.from_scalar(2.0)
    # (plain products: rtol = atol = 1e-2 against the fp32 product; with a bias the product is rounded before it is
    # scaled by alpha = 2 and may be cancelled by the bias, so one ulp of the product sets the absolute tolerance)
    biased = dict(rtol=2e-2, atol=2e-2 * max(k / 512, 1) ** 0.5) if dtype == torch.bfloat16 else dict(rtol=1e-2, atol=1e-2 * max(k / 512, 1) ** 0.5)
    a = torch.randn(m, k, dtype=dtype, device="cuda")
    bias = torch.randn(m, n, dtype=dtype, device="cuda")
    for b in (torch.randn(k, n, dtype=dtype, device="cuda"), torch.randn(n, k, dtype=dtype, device="cuda").t()):
        product = a.float() @ b.float()
        for out_dtype, with_bias in ((dtype, False), (torch.float32, False), (dtype, True)):
            buffer = torch.full((m, n + 8), 7.0, dtype=out_dtype, device="cuda")
            out = buffer[:, :n]
            tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
            expected = 0.5 * bias.float() + 2.0 * product.to(dtype).float() if with_bias else product
            out_tag = runtime.DATA_TYPE_INDEX["fp32"] if out_dtype == torch.float32 else tag
            served = 0
            for instance, name in enumerate(names):
                if "split-k" not in name:
                    continue
                for _ in range(2):
                    out.fill_(float("nan"))
                    result = lib.launch_nt_gemm_config(
                        runtime.current_stream(), instance, tensors[0] if with_bias else null, tensors[1], tensors[2], beta if with_bias else null,
                        alpha if with_bias else null, tensors[3], tag, out_tag,
                    )
                    if result == 1:
                        break
                    assert result == 0, name
                    assert torch.allclose(out.float(), expected, **(biased if with_bias else HALF_TOL)), (name, out_dtype, with_bias)
                    assert bool((buffer[:, n:] == 7.0).all()), name
                else:
                    served += 1
            assert served >= 1 or (n % 8 != 0 and b.stride(1) == 1)
        out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        _matmul_kernel()(a, b, out)
        assert torch.allclose(out.float(), product, **HALF_TOL)
