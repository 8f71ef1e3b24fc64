"""A matrix product followed by element-wise work on the accumulator (bias, activation, scaling,
a residual): not one of the reference's own test programs, but the obvious next thing a user of
`ninetoothed.make` writes after the README's matmul.  The product runs on the GEMM kernels into an
fp32 scratch tensor, the rest as a tile map over it."""

import pytest
import torch

import ninetoothed_amd as ninetoothed
import ninetoothed_amd.language as ntl
from ninetoothed_amd import Tensor, programs


def linear_arrangement(lhs, rhs, bias, residual, scale, output, BM=ninetoothed.block_size(), BN=ninetoothed.block_size(), BK=ninetoothed.block_size()):
    lhs_arranged, rhs_arranged, output_arranged = programs.matmul.arrangement(lhs, rhs, output, BM, BN, BK)
    bias_arranged = bias.tile((BN,)).unsqueeze(0).expand((output_arranged.shape[0], -1))
    return lhs_arranged, rhs_arranged, bias_arranged, residual.tile((BM, BN)), scale, output_arranged


def linear_application(lhs, rhs, bias, residual, scale, output):
    accumulator = ntl.zeros(output.shape, dtype=ntl.float32)
    for k in range(lhs.shape[0]):
        accumulator += ntl.dot(lhs[k], rhs[k])
    activated = ntl.maximum(accumulator * scale + bias[None, :], 0)
    output = activated + residual  # noqa: F841


def _kernel():
    return ninetoothed.make(linear_arrangement, linear_application, (Tensor(2), Tensor(2), Tensor(1), Tensor(2), Tensor(0), Tensor(2)))


def test_recognised_as_a_product_with_an_epilogue():
    kernel = _kernel()
    assert kernel.kind == "gemm_epilogue"
    assert (kernel.details["lhs"], kernel.details["rhs"], kernel.details["output"]) == (0, 1, 5)
    # the epilogue reads the accumulator as a tile of one more tensor, arranged like the output
    text = kernel.details["epilogue"].describe()
    assert "load(ref[6,1,])" in text and "dot" not in text

    def two_products(lhs, rhs, bias, residual, scale, output):
        first = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            first += ntl.dot(lhs[k], rhs[k])
        second = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            second += ntl.dot(lhs[k], rhs[k]) * 2
        output = first + second  # noqa: F841

    with pytest.raises(ninetoothed.UnsupportedProgram):
        ninetoothed.make(linear_arrangement, two_products, (Tensor(2), Tensor(2), Tensor(1), Tensor(2), Tensor(0), Tensor(2)))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16, torch.float32))
@pytest.mark.parametrize("m, n, k", ((512, 384, 256), (300, 200, 136), (1024, 1024, 2048)))
def test_linear_with_bias_activation_and_residual(m, n, k, dtype):
    kernel = _kernel()
    lhs = torch.randn(m, k, dtype=dtype, device="cuda")
    rhs = torch.randn(k, n, dtype=dtype, device="cuda")
    bias = torch.randn(n, dtype=dtype, device="cuda")
    residual = torch.randn(m, n, dtype=dtype, device="cuda")
    scale = 0.125
    expected = (torch.relu(lhs.float() @ rhs.float() * scale + bias.float()) + residual.float()).to(dtype)
    for _ in range(2):
        output = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        kernel(lhs, rhs, bias, residual, scale, output)
        assert "launch_nt_matmul" in kernel.last_plan and "launch_nt_map" in kernel.last_plan
        assert torch.allclose(output.float(), expected.float(), rtol=1e-2, atol=1e-2)
