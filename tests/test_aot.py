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


def test_packaging_needs_element_types(tmp_path):
    with pytest.raises(UnsupportedProgram):
        _package(tmp_path, "untyped", programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())

    def arrangement(x, y):
        return x.tile((256,)), y.tile((256,))

    def application(x, y):
        y = x + 1  # noqa: F841

    with pytest.raises(UnsupportedProgram):
        _package(tmp_path, "add_one", arrangement, application, (Tensor(1), Tensor(1, dtype=ninetoothed.float32)))


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


_CONV_CONFIGS = (
    ((), {"block_size_m": 64, "block_size_n": 64, "block_size_k": 64}, {}),
    ((), {"block_size_m": 128, "block_size_n": 32, "block_size_k": 64}, {}),
)
_CONV_SIZES = {"n": 4, "c": 64, "h": 16, "w": 16, "k": 512, "r": 3, "s": 3}


def _conv2d_premake(constexpr_shapes):
    sizes = _CONV_SIZES if constexpr_shapes else dict.fromkeys(_CONV_SIZES)
    return sizes, functools.partial(programs.conv2d.premake, **sizes, dtype=ninetoothed.float16)


def test_build_writes_a_dispatcher_over_the_configurations(tmp_path):
    """`build` after the reference's src/ninetoothed/build.py:26-170: one launch function whose
    trailing integers select the configuration; 1 when none matches."""
    _, premake = _conv2d_premake(False)
    kernel = ninetoothed.build(premake, _CONV_CONFIGS, caller="hip", kernel_name="conv2d", output_dir=tmp_path)
    assert kernel.config_parameters == ("n_", "c_", "h_", "w_", "k_", "r_", "s_", "dtype_", "block_size_m_", "block_size_n_", "block_size_k_")
    source = (tmp_path / "conv2d.c").read_text()
    assert "NineToothedTensor lhs, NineToothedTensor rhs, NineToothedTensor output, int n_," in source
    assert "dtype_ == 8 && block_size_m_ == 128 && block_size_n_ == 32 && block_size_k_ == 64" in source
    assert source.rstrip().endswith("return 1;\n}")
    packaged = (tmp_path / "conv2d_0_0_0_0_0_0_0_8_128_32_64.c").read_text()
    assert "launch_nt_conv2d(stream, lhs, rhs, output, NINETOOTHED_FLOAT16, 0, 0, 128, 32, 64)" in packaged
    # no configuration matches: the dispatcher returns 1 without touching its tensors
    library = ctypes.CDLL(kernel.library_path)
    from ninetoothed_amd import runtime

    library.launch_conv2d.argtypes = [ctypes.c_void_p] + [runtime.ArgumentTensor] * 3 + [ctypes.c_int] * 11
    null = runtime.ArgumentTensor.null()
    assert library.launch_conv2d(None, null, null, null, *([0] * 7), 8, 32, 32, 32) == 1

    # an unchanged fingerprint reuses the library; a changed configuration rebuilds it
    stamp = (tmp_path / "conv2d.so").stat().st_mtime_ns
    ninetoothed.build(premake, _CONV_CONFIGS, caller="hip", kernel_name="conv2d", output_dir=tmp_path)
    assert (tmp_path / "conv2d.so").stat().st_mtime_ns == stamp
    ninetoothed.build(premake, _CONV_CONFIGS[:1], caller="hip", kernel_name="conv2d", output_dir=tmp_path)
    assert (tmp_path / "conv2d.so").stat().st_mtime_ns != stamp


def test_build_with_meta_parameters_drops_them_and_is_lazy_on_request(tmp_path):
    _, premake = _conv2d_premake(True)
    meta = ("block_size_m", "block_size_n", "block_size_k")
    lazy = ninetoothed.build(premake, _CONV_CONFIGS, meta_parameters=meta, caller="hip", kernel_name="conv2d_tuned", output_dir=tmp_path, lazy=True)
    assert not (tmp_path / "conv2d_tuned.so").exists()
    kernel = ninetoothed.build(premake, _CONV_CONFIGS, meta_parameters=meta, caller="hip", kernel_name="conv2d_tuned", output_dir=tmp_path)
    assert kernel.config_parameters == ("n_", "c_", "h_", "w_", "k_", "r_", "s_", "dtype_")
    packaged = (tmp_path / "conv2d_tuned_4_64_16_16_512_3_3_8.c").read_text()
    assert "NINETOOTHED_FLOAT16, 0, 0, 0, 0, 0)" in packaged  # no block hints: the library chooses
    with pytest.raises(TypeError):
        kernel()
    del lazy


@pytest.mark.gpu
@pytest.mark.parametrize("constexpr_shapes", (False, True))
def test_built_conv2d(tmp_path, constexpr_shapes):
    """The reference's tests/test_aot.py:215-302 with `test_build=True`."""
    sizes, premake = _conv2d_premake(constexpr_shapes)
    kernel = ninetoothed.build(premake, _CONV_CONFIGS, caller="hip", kernel_name="conv2d", output_dir=tmp_path)
    n, c, h, w, k, r, s = _CONV_SIZES.values()
    input = torch.randn(n, c, h, w, dtype=torch.float16, device="cuda")
    filter = torch.randn(k, c, r, s, dtype=torch.float16, device="cuda")
    # fp32 convolution of the same fp16 values: the vendor's fp16 convolution itself differs from it by more than 1e-2 in places
    expected = F.conv2d(input.float(), filter.float()).half()
    for config in _CONV_CONFIGS:
        output = torch.full((n, k, h - r + 1, w - s + 1), float("nan"), dtype=torch.float16, device="cuda")
        kernel(input, filter, output, *sizes.values(), ninetoothed.float16, *config[1].values())
        assert torch.allclose(output, expected, rtol=1e-2, atol=1e-2)
    with pytest.raises(ninetoothed.KernelLaunchError):
        kernel(input, filter, output, *sizes.values(), ninetoothed.float16, 32, 32, 32)
    meta = ("block_size_m", "block_size_n", "block_size_k")
    tuned = ninetoothed.build(premake, _CONV_CONFIGS, meta_parameters=meta, caller="hip", kernel_name="conv2d_tuned", output_dir=tmp_path)
    output = torch.full_like(output, float("nan"))
    tuned(input, filter, output, *sizes.values(), ninetoothed.float16)
    assert torch.allclose(output, expected, rtol=1e-2, atol=1e-2)
    # `make` of one configuration (the `test_build=False` branch of the same reference test)
    single = _package(tmp_path, "conv2d_single", *premake())
    output = torch.full_like(output, float("nan"))
    single(input, filter, output)
    assert torch.allclose(output, expected, rtol=1e-2, atol=1e-2)
