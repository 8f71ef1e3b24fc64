"""Ahead-of-time packaging (`make(..., caller="hip")`), after the reference's
tests/test_aot.py: the packaged dispatcher is built and, on a GPU, called through
ctypes like a downstream C caller would."""

import ctypes
import functools
import pathlib
import subprocess

import pytest
import torch
import torch.nn.functional as F

import ninetoothed_amd as ninetoothed
from ninetoothed_amd import Tensor, programs
from ninetoothed_amd.recognition import UnsupportedProgram


def _package(tmp_path, name, arrangement, application, tensors):
    return ninetoothed.make(arrangement, application, tensors, caller="hip", kernel_name=name, output_dir=tmp_path)


def _addmm_package(tmp_path):
    arrangement = functools.partial(programs.addmm.arrangement, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64)
    tensors = tuple(Tensor(ndim, dtype=ninetoothed.float16) for ndim in (2, 2, 2, 0, 0, 2))
    return _package(tmp_path, "addmm_fp16", arrangement, programs.addmm.application, tensors)


def test_packaging_writes_header_source_and_library(tmp_path):
    kernel = _addmm_package(tmp_path)
    header = (tmp_path / "addmm_fp16.h").read_text()
    source = (tmp_path / "addmm_fp16.c").read_text()
    assert "NineToothedResult launch_addmm_fp16(NineToothedStream stream, NineToothedTensor input, NineToothedTensor mat1" in header
    assert "launch_nt_addmm(stream, input, mat1, mat2, beta, alpha, output, NINETOOTHED_FLOAT16, 64, 64, 64)" in source
    library = ctypes.CDLL(kernel.library_path)
    assert hasattr(library, "launch_addmm_fp16")
    # a C caller links it like any other library
    main = tmp_path / "main.c"
    main.write_text('#include "addmm_fp16.h"\nint main(void) { return launch_addmm_fp16 == 0; }\n')
    include = pathlib.Path(ninetoothed.__file__).resolve().parent.parent / "include"
    lib_dir = pathlib.Path(ninetoothed.__file__).resolve().parent / "lib"
    command = ["gcc", str(main), f"-I{include}", f"-I{tmp_path}", str(tmp_path / "addmm_fp16.so"), f"-L{lib_dir}", "-lnt_hip", f"-Wl,-rpath,{lib_dir}", f"-Wl,-rpath,{tmp_path}", "-o", str(tmp_path / "main")]
    assert subprocess.run(command, capture_output=True, text=True).returncode == 0


def test_packaging_needs_element_types_and_a_recognised_program(tmp_path):
    with pytest.raises(UnsupportedProgram):
        _package(tmp_path, "untyped", programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())

    def arrangement(x, y):
        return x.tile((256,)), y.tile((256,))

    def application(x, y):
        y = x + 1  # noqa: F841

    with pytest.raises(UnsupportedProgram):
        _package(tmp_path, "add_one", arrangement, application, (Tensor(1, dtype=ninetoothed.float32), Tensor(1, dtype=ninetoothed.float32)))


@pytest.mark.gpu
def test_packaged_addmm(tmp_path):
    kernel = _addmm_package(tmp_path)
    m = n = k = 512
    input, mat1, mat2 = (torch.randn(shape, dtype=torch.float16, device="cuda") for shape in ((m, n), (m, k), (k, n)))
    beta, alpha = torch.randn((), dtype=torch.float16), torch.randn((), dtype=torch.float16)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel(input, mat1, mat2, beta, alpha, out)
    assert torch.allclose(out, torch.addmm(input, mat1, mat2, beta=beta.item(), alpha=alpha.item()), atol=0.075)


@pytest.mark.gpu
def test_packaged_matmul_and_attention(tmp_path):
    tensors = tuple(Tensor(2, dtype=ninetoothed.float16) for _ in range(3))
    kernel = _package(tmp_path, "matmul_fp16", programs.matmul.arrangement, programs.matmul.application_with_cast, tensors)
    lhs, rhs = torch.randn(512, 384, dtype=torch.float16, device="cuda"), torch.randn(384, 256, dtype=torch.float16, device="cuda")
    out = torch.full((512, 256), float("nan"), dtype=torch.float16, device="cuda")
    kernel(lhs, rhs, out)
    assert torch.allclose(out, torch.matmul(lhs, rhs), rtol=1e-2, atol=1e-2)

    options = (None, None, {"constexpr": True}, {"constexpr": True, "upper_bound": 128})
    q_, k_, v_, o_ = (Tensor(4, dtype=ninetoothed.float16, shape_options=options) for _ in range(4))
    tensors = (q_, k_, v_, Tensor(0, constexpr=True), o_)
    kernel = _package(tmp_path, "attention_fp16", programs.attention.arrangement, programs.attention.application, tensors)
    q, k, v = (torch.randn(2, 4, 1024, 64, dtype=torch.float16, device="cuda") for _ in range(3))
    o = torch.full_like(q, float("nan"))
    kernel(q, k, v, torch.tensor(True), o)
    assert torch.allclose(o, F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=1), rtol=1e-2, atol=1e-2)
