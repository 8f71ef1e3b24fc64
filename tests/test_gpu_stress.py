"""Whole-output checks at the baseline shapes, repeated on outputs that start as
NaN: a synchronisation mistake in a pipelined kernel shows up as a few wrong rows
in a few tiles and only under load, which sampled rows of a large problem or small
problems do not see.  Every launch must also reproduce itself bit for bit (no
kernel here reduces in a data-dependent order)."""

import ctypes

import pytest
import torch
import torch.nn.functional as F

import ninetoothed_amd as ninetoothed
from ninetoothed_amd import programs, runtime

pytestmark = pytest.mark.gpu

HALF_TOL = dict(rtol=1e-2, atol=1e-2)


def _seeded(*shape, dtype=torch.float16, scale=1.0, seed=0):
    generator = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=generator) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_addmm_8192_whole_output_and_repeatability(dtype):
    n = 8192
    input, mat1, mat2 = _seeded(n, n, dtype=dtype, seed=0), _seeded(n, n, dtype=dtype, seed=1), _seeded(n, n, dtype=dtype, scale=0.05, seed=2)
    application = programs.addmm.application if dtype == torch.float16 else programs.addmm.application_bfloat16
    kernel = ninetoothed.make(programs.addmm.arrangement, application, programs.addmm.tensors())
    expected = torch.addmm(input, mat1, mat2, beta=0.5, alpha=1.0)
    first = None
    for _ in range(3):
        out = torch.full((n, n), float("nan"), dtype=dtype, device="cuda")
        kernel(input, mat1, mat2, 0.5, 1.0, out)
        assert kernel.last_plan.startswith("launch_nt_addmm")
        assert torch.allclose(out, expected, rtol=2e-2, atol=2e-2)
        if first is None:
            first = out
        else:
            assert torch.equal(out, first)


def test_every_gemm_instance_whole_output():
    lib = runtime.library()
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    n = 2048
    a, b = _seeded(n, n, seed=3), _seeded(n, n, scale=0.05, seed=4)
    expected = torch.matmul(a, b)
    null = runtime.ArgumentTensor.null()
    ran = 0
    for config in range(lib.nt_gemm_num_configs()):
        for _ in range(2):
            out = torch.full((n, n), float("nan"), dtype=torch.float16, device="cuda")
            code = lib.launch_nt_gemm_config(
                runtime.current_stream(), config, null, runtime.ArgumentTensor.from_torch_tensor(a), runtime.ArgumentTensor.from_torch_tensor(b),
                null, null, runtime.ArgumentTensor.from_torch_tensor(out), fp16, fp16,
            )
            if code == 1 and "split-k" in runtime.gemm_config_names()[config]:
                break  # takes problems with few output tiles only (tests/test_gpu_parity.py::test_gemm_split_k)
            assert code == 0, runtime.gemm_config_names()[config]
            assert torch.allclose(out, expected, **HALF_TOL), runtime.gemm_config_names()[config]
        else:
            ran += 1
    assert ran >= sum("split-k" not in name for name in runtime.gemm_config_names())


def test_conv2d_baseline_whole_output_and_repeatability():
    x = _seeded(32, 256, 56, 56, scale=0.1, seed=5)
    w = _seeded(256, 256, 3, 3, scale=0.1, seed=6)
    kernel = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    expected = F.conv2d(x, w, padding=1)
    first = None
    for _ in range(3):
        out = torch.full((32, 256, 56, 56), float("nan"), dtype=torch.float16, device="cuda")
        kernel(x, w, out, padding_h=1, padding_w=1)
        assert torch.allclose(out, expected, **HALF_TOL)
        if first is None:
            first = out
        else:
            assert torch.equal(out, first)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("head_dim", (64, 128))
@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_whole_output_and_repeatability(is_causal, head_dim, dtype):
    shape = (4, 16, 4096 if head_dim == 128 else 2048 + 64, head_dim)
    q, k, v = (_seeded(*shape, dtype=dtype, seed=s) for s in (7, 8, 9))
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
    expected = torch.cat([F.scaled_dot_product_attention(q[b : b + 1], k[b : b + 1], v[b : b + 1], is_causal=is_causal, scale=head_dim**-0.5) for b in range(4)])
    tolerance = HALF_TOL if dtype == torch.float16 else dict(rtol=2e-2, atol=2e-2)
    first = None
    for _ in range(3):
        out = torch.full_like(q, float("nan"))
        kernel(q, k, v, is_causal, head_dim**-0.5, out)
        assert torch.allclose(out, expected, **tolerance)
        if first is None:
            first = out
        else:
            assert torch.equal(out, first)


def test_softmax_baseline_whole_output():
    x = _seeded(4096, 4096, dtype=torch.float32, seed=10)
    kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    expected = torch.softmax(x, dim=-1)
    for _ in range(3):
        out = torch.full_like(x, float("nan"))
        kernel(x, out, BLOCK_SIZE=4096)
        assert torch.allclose(out, expected, rtol=1e-5, atol=1e-6)
