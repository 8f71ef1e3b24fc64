"""``launch_nt_matmul_static_scratch``: the matmul entry point that allocates nothing (split-K partial
products go to a fixed array inside the library) against ``launch_nt_matmul``, through the C ABI, on two
calls in a row -- the second with a smaller input, so it runs on what the first one left in the array --
bit for bit: both entry points run the same kernels with the same split."""

import pytest
import torch

from ninetoothed_amd import runtime

pytestmark = pytest.mark.gpu


def _operands(m, n, k, dtype, seed):
    generator = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=generator).to(dtype).cuda()
    b = (torch.randn(k, n, generator=generator) * 0.1).to(dtype).cuda()
    return a, b


def _call(entry, a, b, out, dtype_tag, out_tag="same"):
    tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (a, b, out)]
    dtype = runtime.DATA_TYPE_INDEX[dtype_tag]
    out_dtype = dtype if out_tag == "same" else runtime.DATA_TYPE_INDEX[out_tag]
    return entry(runtime.current_stream(), tensors[0], tensors[1], tensors[2], dtype, out_dtype, 0, 0, 0)


@pytest.mark.parametrize("dtype, tag", ((torch.float16, "fp16"), (torch.bfloat16, "bf16")))
def test_static_scratch_matmul_matches_the_allocating_entry_point(dtype, tag):
    lib = runtime.library()
    # split-K problems (few output tiles, long K); partial products: 4 x 16 x 8192 and 32 x 16 x 1024 floats = 2 MiB each
    problems = ((16, 8192, 8192), (16, 1024, 4096), (100, 520, 4104))
    print("static-scratch matmul", tag, problems, flush=True)
    warm_a, warm_b = _operands(256, 256, 256, dtype, 1)
    warm = torch.empty(256, 256, dtype=dtype, device="cuda")
    assert _call(lib.launch_nt_matmul_static_scratch, warm_a, warm_b, warm, tag) == 0  # code objects and the array are resident from here on
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    outputs = []
    for index, (m, n, k) in enumerate(problems):
        a, b = _operands(m, n, k, dtype, 10 + index)
        out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        outputs.append((a, b, out))
    free_before = torch.cuda.mem_get_info()[0]
    for a, b, out in outputs:
        assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, tag) == 0
    torch.cuda.synchronize()
    # a workspace for these calls would have taken 2 MiB or more from the device
    assert free_before - torch.cuda.mem_get_info()[0] < (1 << 20)
    for a, b, out in outputs:
        expected = torch.full_like(out, float("nan"))
        assert _call(lib.launch_nt_matmul, a, b, expected, tag) == 0
        torch.cuda.synchronize()
        assert torch.equal(out, expected), tuple(out.shape)
        assert torch.allclose(out.float(), a.float() @ b.float(), rtol=1e-2, atol=1e-2)


def test_static_scratch_matmul_fp32_output_one_pass_problems_and_the_limit(tmp_path):
    import csv
    import ctypes

    lib = runtime.library()
    print("static-scratch matmul: fp32 output, one-pass problem, scratch limit", flush=True)
    a, b = _operands(64, 2048, 8192, torch.float16, 20)
    out, expected = (torch.full((64, 2048), float("nan"), dtype=torch.float32, device="cuda") for _ in range(2))
    assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, "fp16", "fp32") == 0
    assert _call(lib.launch_nt_matmul, a, b, expected, "fp16", "fp32") == 0
    torch.cuda.synchronize()
    assert torch.equal(out, expected)
    # a problem with enough tiles runs in one pass and needs no scratch memory: any size goes
    a, b = _operands(2048, 2048, 512, torch.float16, 21)
    out, expected = (torch.full((2048, 2048), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2))
    assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, "fp16") == 0
    assert _call(lib.launch_nt_matmul, a, b, expected, "fp16") == 0
    torch.cuda.synchronize()
    assert torch.equal(out, expected)
    # 32 parts x 512 x 512 floats = 32 MiB of partial products do not fit the 16 MiB array: the call runs with the 16
    # parts that do (another summation order than launch_nt_matmul's 32 parts, so equal within rounding only)
    a, b = _operands(512, 512, 65536, torch.float16, 22)
    out, expected = (torch.full((512, 512), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2))
    assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, "fp16") == 0
    assert _call(lib.launch_nt_matmul, a, b, expected, "fp16") == 0
    torch.cuda.synchronize()
    assert torch.allclose(out.float(), expected.float(), rtol=1e-2, atol=1e-2)
    # 1024 x 2560 outputs: 64 x 64 tiles fill the chip, so the untuned choice is one pass and any size goes
    a, b = _operands(1024, 2560, 8192, torch.float16, 23)
    out, expected = (torch.full((1024, 2560), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2))
    assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, "fp16") == 0
    assert "split-k" not in runtime.last_launch(), runtime.last_launch()
    assert _call(lib.launch_nt_matmul, a, b, expected, "fp16") == 0
    torch.cuda.synchronize()
    assert torch.equal(out, expected)
    # ... until a tuned choice names a split-K instance for the problem (here: read from a cache file): even two parts
    # of partial products (20 MiB) exceed the array -> refused, nothing written
    names = runtime.gemm_config_names()
    split = next(i for i, name in enumerate(names) if name.startswith("256x256x32") and "split-k" in name)
    fp16 = runtime.DATA_TYPE_INDEX["fp16"]
    path = tmp_path / "tuned.csv"
    with open(path, "w", newline="") as handle:
        writer = csv.writer(handle)
        writer.writerow(())
        writer.writerow((lib.nt_tune_file_format(),))
        writer.writerow((runtime.TUNE_GEMM, fp16, fp16, 1024, 2560, 8192, 0, 0))
        writer.writerow((split, 256, 256, 32))
    entries = ctypes.c_int(0)
    assert lib.nt_tune_cache_load(str(path).encode(), ctypes.byref(entries)) == 0 and entries.value == 1
    out.fill_(float("nan"))
    assert _call(lib.launch_nt_matmul_static_scratch, a, b, out, "fp16") == runtime.SCRATCH_LIMIT
    torch.cuda.synchronize()
    assert bool(torch.isnan(out).all())
    assert _call(lib.launch_nt_matmul, a, b, out, "fp16") == 0  # (with the stream's buffer the tuned instance runs)
    assert "split-k" in runtime.last_launch(), runtime.last_launch()
    torch.cuda.synchronize()
    assert torch.allclose(out.float(), expected.float(), rtol=1e-2, atol=1e-2 * 4)
    assert runtime.STATIC_SCRATCH_BYTES == 16 << 20


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
def test_static_scratch_matmul_never_takes_buffers_for_copies():
    """fp8 operands and operands the direct-to-LDS kernels cannot read in place run on copies in allocated buffers
    under ``launch_nt_matmul``; the entry point that allocates nothing must take the kernels that read them in place."""
    lib = runtime.library()
    print("static-scratch matmul: fp8 and misaligned operands, no buffers", flush=True)
    lib.nt_release_workspaces()
    m, n, k = 2056, 1032, 1040  # 2^31 multiply-adds and more
    a8 = torch.randn(m, k, device="cuda").to(torch.float8_e5m2)
    b8 = torch.randn(k, n, device="cuda").to(torch.float8_e5m2)
    a_off = torch.randn(m, k + 1, dtype=torch.float16, device="cuda")[:, :k]
    b16 = torch.randn(k, n, dtype=torch.float16, device="cuda")
    out8, out16 = (torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert _call(lib.launch_nt_matmul_static_scratch, a8, b8, out8, "fp8e5m2", "fp16") == 0
    assert "any-stride" in runtime.last_launch(), runtime.last_launch()
    assert _call(lib.launch_nt_matmul_static_scratch, a_off, b16, out16, "fp16") == 0
    assert "any-stride" in runtime.last_launch(), runtime.last_launch()
    torch.cuda.synchronize()
    assert free_before - torch.cuda.mem_get_info()[0] < (1 << 20)  # (the copies would have taken 8 MiB and more)
    tolerance = dict(rtol=1e-2, atol=1e-2 * (k / 512) ** 0.5)
    assert torch.allclose(out8.float(), a8.to(torch.float16).float() @ b8.to(torch.float16).float(), **tolerance)
    assert torch.allclose(out16.float(), a_off.float() @ b16.float(), **tolerance)
    # fp32 products of few tiles and products a few tiles over whole rounds of the chip put partial products into
    # allocated buffers under launch_nt_matmul; here they run in one pass
    print("static-scratch matmul: fp32 products of few tiles, 17 x 17 tiles, no buffers", flush=True)
    lib.nt_release_workspaces()
    a32, b32 = torch.randn(128, 4096, device="cuda"), torch.randn(4096, 128, device="cuda")
    out32 = torch.full((128, 128), float("nan"), device="cuda")
    big_a, big_b = torch.randn(4352, 2048, dtype=torch.float16, device="cuda"), torch.randn(2048, 4352, dtype=torch.float16, device="cuda") * 0.1
    big_out = torch.full((4352, 4352), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert _call(lib.launch_nt_matmul_static_scratch, a32, b32, out32, "fp32") == 0
    assert "parts" not in runtime.last_launch(), runtime.last_launch()
    assert _call(lib.launch_nt_matmul_static_scratch, big_a, big_b, big_out, "fp16") == 0
    assert "last rows" not in runtime.last_launch(), runtime.last_launch()
    torch.cuda.synchronize()
    assert free_before - torch.cuda.mem_get_info()[0] < (1 << 20)
    assert torch.allclose(out32.double(), a32.double() @ b32.double(), rtol=1e-4, atol=1e-3)
    assert torch.allclose(big_out.float(), big_a.float() @ big_b.float(), rtol=1e-2, atol=2e-2)
