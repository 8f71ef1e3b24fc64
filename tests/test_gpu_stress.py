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
    # the program's arithmetic in fp32: product rounded to the element type, combined in fp32, rounded once
    product = (mat1.float() @ mat2.float()).to(dtype).float()
    expected = (0.5 * input.float() + product).to(dtype)
    # fp16: rtol = atol = 1e-2.  bf16: two correct fp32 sums may round to neighbouring bf16 products, one ulp apart
    # (2^-7 of a product of magnitude up to ~16 here = 0.06 at most, typically 0.03), and the input term may cancel
    # the rest of the value: the absolute tolerance is one bf16 ulp of the typical product, not a hundredth.
    tolerance = dict(rtol=1e-2, atol=1e-2) if dtype == torch.float16 else dict(rtol=1e-2, atol=2.0**-7 * float(product.abs().max()))
    del product
    vendor = torch.addmm(input, mat1, mat2, beta=0.5, alpha=1.0)
    first = None
    for _ in range(3):
        out = torch.full((n, n), float("nan"), dtype=dtype, device="cuda")
        kernel(input, mat1, mat2, 0.5, 1.0, out)
        assert kernel.last_plan.startswith("launch_nt_addmm")
        assert torch.allclose(out, expected, **tolerance)
        assert torch.allclose(out, vendor, rtol=2e-2, atol=2e-2 if dtype == torch.float16 else tolerance["atol"])
        if first is None:
            first = out
        else:
            assert torch.equal(out, first)


def test_addmm_8192_at_the_stated_input_distribution():
    """All three operands N(0, 1), alpha = 1.0, beta = 0.5 (the inputs the throughput figure is quoted
    on): whole output against the program's arithmetic done by torch in fp32 -- product rounded to
    fp16, combined in fp32, rounded once -- at rtol = atol = 1e-2, and against ``torch.addmm``."""
    n = 8192
    input, mat1, mat2 = (_seeded(n, n, seed=seed) for seed in (10, 11, 12))
    kernel = ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())
    out = torch.full((n, n), float("nan"), dtype=torch.float16, device="cuda")
    kernel(input, mat1, mat2, 0.5, 1.0, out)
    assert kernel.last_plan.startswith("launch_nt_addmm")
    product = (mat1.float() @ mat2.float()).half().float()
    expected = (0.5 * input.float() + 1.0 * product).half()
    del product
    assert torch.allclose(out, expected, **HALF_TOL)
    assert torch.allclose(out, torch.addmm(input, mat1, mat2, beta=0.5, alpha=1.0), rtol=1e-2, atol=0.075)  # reference tolerance, tests/test_addmm.py:59


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
    expected = F.conv2d(x.float(), w.float(), padding=1)  # fp32 convolution of the same operands
    vendor = F.conv2d(x, w, padding=1)
    first = None
    for _ in range(3):
        out = torch.full((32, 256, 56, 56), float("nan"), dtype=torch.float16, device="cuda")
        kernel(x, w, out, padding_h=1, padding_w=1)
        assert torch.allclose(out.float(), expected, **HALF_TOL)
        assert torch.allclose(out, vendor, **HALF_TOL)  # the stock fp16 operator of the same GPU
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
    # fp32 attention on the same (rounded) operands, four heads at a time, at rtol = atol = 1e-2 for both types;
    # the stock operator of the same GPU as a second check (bf16: its output is two bf16 roundings away)
    seq = shape[2]
    mask = torch.ones(seq, seq, dtype=torch.bool, device="cuda").tril() if is_causal else None

    def reference(qs, ks, vs):
        scores = (qs.float() * head_dim**-0.5) @ ks.float().transpose(-1, -2)
        if mask is not None:
            scores = scores.masked_fill(~mask, float("-inf"))
        return torch.softmax(scores, dim=-1) @ vs.float()

    expected = torch.cat([torch.cat([reference(q[b : b + 1, h : h + 4], k[b : b + 1, h : h + 4], v[b : b + 1, h : h + 4]) for h in range(0, 16, 4)], dim=1) for b in range(4)])
    vendor = torch.cat([F.scaled_dot_product_attention(q[b : b + 1], k[b : b + 1], v[b : b + 1], is_causal=is_causal, scale=head_dim**-0.5) for b in range(4)])
    vendor_tolerance = HALF_TOL if dtype == torch.float16 else dict(rtol=2e-2, atol=2e-2)
    first = None
    for _ in range(3):
        out = torch.full_like(q, float("nan"))
        kernel(q, k, v, is_causal, head_dim**-0.5, out)
        assert torch.allclose(out.float(), expected, **HALF_TOL)
        assert torch.allclose(out, vendor, **vendor_tolerance)
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


def test_gemm_instances_on_random_shapes():
    """Every instance on 48 seeded random problems: any M, N and K with and without the divisibility the
    direct-to-LDS kernels ask for, both rhs layouts, padded row pitches, element-type / fp32 / addmm
    outputs.  An instance either declines (1) or writes the whole NaN-poisoned output correctly and
    leaves the sentinels around it alone."""
    import random

    lib = runtime.library()
    names = runtime.gemm_config_names()
    null = runtime.ArgumentTensor.null()
    fp16, fp32 = runtime.DATA_TYPE_INDEX["fp16"], runtime.DATA_TYPE_INDEX["fp32"]
    beta, alpha = runtime.ArgumentTensor.from_scalar(-0.75), runtime.ArgumentTensor.from_scalar(1.5)
    rng = random.Random(20240607)
    served = {name: 0 for name in names}
    for case in range(48):
        m = rng.choice((1, 3, 16, 64, 100, 129, 256, 300, 513, 700))
        n = rng.choice((8, 24, 64, 72, 128, 200, 256, 264, 520, 1000)) + rng.choice((0, 0, 0, 1, 5))
        k = rng.choice((8, 16, 64, 72, 256, 520, 1024, 2056, 4096)) + rng.choice((0, 0, 0, 3))
        transposed = rng.random() < 0.5
        pad_a, pad_b, pad_c = (rng.choice((0, 0, 8, 24)) for _ in range(3))
        a = torch.randn(m, k + pad_a, dtype=torch.float16, device="cuda")[:, :k]
        if transposed:
            b = torch.randn(n, k + pad_b, dtype=torch.float16, device="cuda")[:, :k].t()
        else:
            b = torch.randn(k, n + pad_b, dtype=torch.float16, device="cuda")[:, :n]
        bias = torch.randn(m, n, dtype=torch.float16, device="cuda")
        product = a.float() @ b.float()
        mode = rng.choice(("plain", "fp32", "addmm"))
        out_dtype = torch.float32 if mode == "fp32" else torch.float16
        buffer = torch.full((m + 1, n + pad_c + 8), 7.0, dtype=out_dtype, device="cuda")
        out = buffer[:m, :n]
        expected = -0.75 * bias.float() + 1.5 * product.half().float() if mode == "addmm" else product
        tensors = [runtime.ArgumentTensor.from_torch_tensor(t) for t in (bias, a, b, out)]
        tolerance = dict(rtol=1e-2, atol=1e-2 * max(k / 512, 1) ** 0.5 * (2.0 if mode == "addmm" else 1.0))
        ran = 0
        for instance, name in enumerate(names):
            out.fill_(float("nan"))
            code = lib.launch_nt_gemm_config(
                runtime.current_stream(), instance, tensors[0] if mode == "addmm" else null, tensors[1], tensors[2],
                beta if mode == "addmm" else null, alpha if mode == "addmm" else null, tensors[3], fp16, fp32 if mode == "fp32" else fp16,
            )
            if code == 1:
                continue
            description = (case, m, n, k, transposed, mode, name)
            assert code == 0, description
            assert torch.allclose(out.float(), expected, **tolerance), description
            assert bool((buffer[:m, n:] == 7.0).all()) and bool((buffer[m] == 7.0).all()), description
            served[name] += 1
            ran += 1
        assert ran >= 1, (case, m, n, k, transposed, mode)
    # (the instances without tails need N and K to fit their tiles; test_every_gemm_instance_whole_output covers them)
    assert all(count > 0 for name, count in served.items() if "tails" in name or "any-stride" in name), served


def test_conv2d_on_random_layers():
    """40 seeded random layers: channel counts with and without the multiples the implicit-GEMM kernel
    likes, odd feature maps, filters from 1 x 1 to 5 x 3, every padding that leaves an output; the
    whole NaN-poisoned output against an fp32 convolution, sentinels behind it untouched."""
    import random

    rng = random.Random(777)
    kernel = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    for case in range(40):
        n = rng.choice((1, 2, 3, 8, 33))
        c = rng.choice((1, 3, 8, 16, 32, 40, 64, 96, 136))
        k = rng.choice((8, 16, 24, 64, 72, 128, 200, 256, 320)) + rng.choice((0, 0, 0, 4))
        h, w = rng.choice((7, 8, 13, 14, 28, 31)), rng.choice((7, 8, 12, 14, 28, 33))
        r, s = rng.choice((1, 1, 2, 3, 3, 5)), rng.choice((1, 1, 3, 3))
        pad = (rng.choice((0, 1, 2)), rng.choice((0, 1, 2)))
        if h + 2 * pad[0] < r or w + 2 * pad[1] < s:
            continue
        x = (torch.randn(n, c, h, w, device="cuda") * 0.5).half()
        weight = (torch.randn(k, c, r, s, device="cuda") * 0.1).half()
        p_out, q_out = h + 2 * pad[0] - r + 1, w + 2 * pad[1] - s + 1
        count = n * k * p_out * q_out
        guard = torch.full((count + 64,), 7.0, dtype=torch.float16, device="cuda")
        out = guard[:count].view(n, k, p_out, q_out)
        out.fill_(float("nan"))
        kernel(x, weight, out, padding_h=pad[0], padding_w=pad[1])
        expected = F.conv2d(x.float(), weight.float(), padding=pad)
        description = (case, n, c, h, w, k, r, s, pad)
        assert torch.allclose(out.float(), expected, rtol=1e-2, atol=1e-2), description
        assert bool((guard[count:] == 7.0).all()), description


def test_attention_on_random_shapes():
    """40 seeded random problems: head dimensions that are any multiple of 8 up to 256, query and key
    lengths from 1 to a few thousand (few or many groups, so with and without a split key range),
    causal where the lengths agree, fp16 and bf16, strided layouts."""
    import random

    rng = random.Random(4242)
    kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
    for case in range(40):
        batch, heads = rng.choice((1, 1, 2, 5)), rng.choice((1, 2, 3, 16))
        emb_dim = rng.choice((8, 32, 40, 64, 64, 96, 128, 128, 160, 256))
        seq_k = rng.choice((1, 17, 64, 200, 513, 1024, 3000, 6000))
        seq_q = seq_k if rng.random() < 0.5 else rng.choice((1, 5, 130, 700))
        is_causal = seq_q == seq_k and rng.random() < 0.5
        dtype = rng.choice((torch.float16, torch.bfloat16))
        packed = rng.random() < 0.3  # [batch, seq, heads, dim] storage viewed as [batch, heads, seq, dim]

        def tensor(seq):
            if packed:
                return (torch.randn(batch, seq, heads, emb_dim, device="cuda") * 0.5).to(dtype).permute(0, 2, 1, 3)
            return (torch.randn(batch, heads, seq, emb_dim, device="cuda") * 0.5).to(dtype)

        q, k, v = tensor(seq_q), tensor(seq_k), tensor(seq_k)
        o = torch.full((batch, heads, seq_q, emb_dim), float("nan"), dtype=dtype, device="cuda")
        scale = emb_dim**-0.5
        kernel(q, k, v, is_causal, scale, o)
        scores = (q.float() * scale) @ k.float().transpose(-1, -2)
        if is_causal:
            scores = scores.masked_fill(~torch.ones(seq_q, seq_k, dtype=torch.bool, device="cuda").tril(), float("-inf"))
        expected = torch.softmax(scores, dim=-1) @ v.float()
        assert torch.allclose(o.float(), expected, **HALF_TOL), (case, batch, heads, seq_q, seq_k, emb_dim, is_causal, dtype, packed)


def test_mfma_rate_probe_runs_and_counts():
    """The measurement aid behind bench.py's ``mfma_ceiling`` workloads: launches, reports the MFMAs it issued
    (8 waves per compute unit x loops x 8; x 32 in the 16x16x32 form) and leaves its sink untouched."""
    import ctypes

    import bench
    from ninetoothed_amd import runtime

    a = torch.randn(64, 64, dtype=torch.float16, device="cuda")
    sink = torch.zeros(1, device="cuda")
    count = ctypes.c_int64(0)
    lib = bench.load_probe_library()  # (a library of its own: the product library does not export measurement aids)
    assert not hasattr(runtime.library(), "nt_probe_mfma_rate")
    tensor = runtime.ArgumentTensor.from_torch_tensor(a)
    runtime.check(lib.nt_probe_mfma_rate(runtime.current_stream(), tensor, tensor, 3, sink.data_ptr(), ctypes.byref(count)))
    torch.cuda.synchronize()
    units = torch.cuda.get_device_properties(0).multi_processor_count
    assert count.value == units * 8 * 3 * 8
    assert sink.item() == 0.0
    small = runtime.ArgumentTensor.from_torch_tensor(a[:8, :8].contiguous())
    assert lib.nt_probe_mfma_rate(runtime.current_stream(), small, small, 3, sink.data_ptr(), ctypes.byref(count)) != 0
    runtime.check(lib.nt_probe_mfma_rate_16x16x32(runtime.current_stream(), tensor, tensor, 3, sink.data_ptr(), ctypes.byref(count)))
    torch.cuda.synchronize()
    assert count.value == units * 8 * 3 * 32
    assert sink.item() == 0.0
    assert lib.nt_probe_mfma_rate_16x16x32(runtime.current_stream(), small, small, 3, sink.data_ptr(), ctypes.byref(count)) != 0


@pytest.mark.skipif(not hasattr(torch, "float8_e5m2"), reason="this torch has no float8_e5m2")
def test_calls_that_share_scratch_buffers_from_several_host_threads():
    """Split-K partial products (of the fp16 and the fp32 kernels), the fp16 copies of fp8 operands, dense copies of
    misaligned operands, padded copies of attention tensors, conv2d's repacked operands and the per-part maxima and sums
    of a softmax over a few long rows all live in one buffer per (device, stream, purpose).  Four
    host threads enqueue such calls onto the SAME stream with sizes of their own: the registry lock must keep a
    call's copies and the kernel that reads them together (a buffer overwritten in between shows as wrong values),
    also when a buffer has to grow in the middle."""
    import threading

    stream = torch.cuda.current_stream()
    matmul = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
    attention = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(with_scale=True))
    conv = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
    softmax = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
    failures = []

    def worker(seed):
        try:
            with torch.cuda.stream(stream):
                generator = torch.Generator(device="cuda").manual_seed(seed)

                def randn(*shape, dtype=torch.float16, scale=1.0):
                    return (torch.randn(*shape, device="cuda", generator=generator) * scale).to(dtype)

                m = 1024 + 256 * seed
                skinny_a, skinny_b = randn(16, 4096 + 512 * seed), randn(4096 + 512 * seed, 2048)  # few tiles, long K: split K
                a8, b8 = randn(m, 512).to(torch.float8_e5m2), randn(512, 768).to(torch.float8_e5m2)
                a_off, b16 = randn(2048 + 8 * seed, 1025)[:, :1024], randn(1024, 1024)  # rows off 16-byte boundaries, 2^31 multiply-adds
                q, k, v = (randn(1, 2 + seed, 96, 20 + 4 * seed) for _ in range(3))
                x, w = randn(2, 3 + seed, 20, 24, scale=0.3), randn(16, 3 + seed, 3, 3, scale=0.3)
                a32, b32 = randn(100 + seed, 2048 + 64 * seed, dtype=torch.float32), randn(2048 + 64 * seed, 130, dtype=torch.float32)  # one tile row of the fp32 kernel: k range in parts
                rows = randn(2 + seed, 100000 + 4096 * seed, dtype=torch.float32)  # a few long rows: parts of a row on workgroups of their own
                expected = (
                    skinny_a.float() @ skinny_b.float(),
                    a8.to(torch.float16).float() @ b8.to(torch.float16).float(),
                    a_off.float() @ b16.float(),
                    torch.softmax((q.float() * q.shape[-1] ** -0.5) @ k.float().transpose(-1, -2), dim=-1) @ v.float(),
                    F.conv2d(x.float(), w.float(), padding=1),
                    (a32.double() @ b32.double()).float(),
                    torch.softmax(rows, dim=-1),
                )
                for _ in range(6):
                    outs = (
                        torch.full((16, 2048), float("nan"), dtype=torch.float16, device="cuda"),
                        torch.full((m, 768), float("nan"), dtype=torch.float16, device="cuda"),
                        torch.full((a_off.shape[0], 1024), float("nan"), dtype=torch.float16, device="cuda"),
                        torch.full_like(q, float("nan")),
                        torch.full((2, 16, 20, 24), float("nan"), dtype=torch.float16, device="cuda"),
                        torch.full((a32.shape[0], 130), float("nan"), dtype=torch.float32, device="cuda"),
                        torch.full_like(rows, float("nan")),
                    )
                    matmul(skinny_a, skinny_b, outs[0])
                    matmul(a8, b8, outs[1])
                    matmul(a_off, b16, outs[2])
                    attention(q, k, v, False, q.shape[-1] ** -0.5, outs[3])
                    conv(x, w, outs[4], padding_h=1, padding_w=1)
                    matmul(a32, b32, outs[5])
                    softmax(rows, outs[6], BLOCK_SIZE=1 << 17)
                    tolerances = (dict(rtol=1e-2, atol=1e-2 * (skinny_a.shape[1] / 512) ** 0.5), dict(rtol=1e-2, atol=1e-2), dict(rtol=1e-2, atol=1e-2 * 2**0.5), HALF_TOL, HALF_TOL,
                                  dict(rtol=1e-4, atol=2e-4), dict(rtol=1e-5, atol=1e-8))
                    for index, (out, reference, tolerance) in enumerate(zip(outs, expected, tolerances)):
                        if not torch.allclose(out.float(), reference, **tolerance):
                            failures.append((seed, index, float((out.float() - reference).abs().max())))
                            return
        except Exception as error:  # noqa: BLE001  (a worker's exception must fail the test, not vanish with its thread)
            failures.append((seed, repr(error)))

    threads = [threading.Thread(target=worker, args=(seed,)) for seed in range(4)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    torch.cuda.synchronize()
    assert not failures, failures
