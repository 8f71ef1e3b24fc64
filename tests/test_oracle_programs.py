"""Pins the CPU restatement of the five programs (oracle/programs.py) against
the library routines the reference's own tests use as their oracle (with the
tolerances those tests state) and against closed forms chosen so that a dropped
term, a wrong sign or index, or a transposed operand fails."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import programs as oracle


def _half(*shape, scale=1.0):
    return (torch.randn(*shape) * scale).to(torch.float16)


def test_matmul_against_torch():
    # reference: tests/test_matmul.py:67-88 (fp16, compared with torch.matmul)
    a, b = _half(96, 80), _half(80, 72)
    out = oracle.matmul(a.numpy(), b.numpy(), bm=32, bn=16, bk=32)
    expected = torch.matmul(a.float(), b.float()).to(torch.float16).float().numpy()
    assert np.allclose(out, expected, rtol=1e-3, atol=1e-3)


def test_matmul_ragged_blocks_and_identity():
    a = _half(37, 29)
    eye = torch.eye(29, dtype=torch.float16)
    out = oracle.matmul(a.numpy(), eye.numpy(), bm=16, bn=8, bk=4)
    assert np.array_equal(out, a.float().numpy())  # A @ I == A exactly
    # transposed operands would fail here: (2x3) @ (3x4)
    a = np.arange(6, dtype=np.float16).reshape(2, 3)
    b = np.arange(12, dtype=np.float16).reshape(3, 4)
    assert np.array_equal(oracle.matmul(a, b, 2, 2, 2), a.astype(np.float32) @ b.astype(np.float32))


def test_addmm_against_torch():
    # reference: tests/test_addmm.py:57-90 (atol 0.075)
    input, mat1, mat2 = _half(64, 48), _half(64, 40), _half(40, 48)
    beta, alpha = 0.37, 0.81
    out = oracle.addmm(input.numpy(), mat1.numpy(), mat2.numpy(), beta, alpha, 32, 16, 8)
    expected = torch.addmm(input.float(), mat1.float(), mat2.float(), beta=beta, alpha=alpha).numpy()
    assert np.allclose(out, expected, atol=0.075)
    # beta and alpha are not swapped, and the product is rounded before scaling
    zero = np.zeros((4, 4), dtype=np.float16)
    ones = np.ones((4, 4), dtype=np.float16)
    assert np.array_equal(oracle.addmm(ones, zero, zero, 0.5, 3.0, 2, 2, 2), np.full((4, 4), 0.5, dtype=np.float32))
    assert np.array_equal(oracle.addmm(zero, ones, np.eye(4, dtype=np.float16), 0.5, 3.0, 2, 2, 2), np.full((4, 4), 3.0, dtype=np.float32))


def test_softmax_against_torch():
    # reference: tests/test_softmax.py:30-40 (fp32 [1823, 781] there; smaller here, default allclose)
    x = torch.rand(183, 781)
    out = oracle.softmax(x.numpy())
    assert np.allclose(out, torch.softmax(x, dim=-1).numpy())
    assert np.allclose(out.sum(axis=1), 1.0, atol=1e-5)
    shifted = oracle.softmax((x + 3.0).numpy())
    assert np.allclose(out, shifted, atol=1e-6)  # shift invariance
    assert np.allclose(oracle.softmax(np.zeros((2, 5), dtype=np.float32)), 0.2)


def test_softmax_blocks_smaller_than_rows_normalise_per_block():
    x = torch.randn(3, 10).numpy()
    out = oracle.softmax(x, block_size=4)
    for start in (0, 4, 8):
        part = torch.softmax(torch.from_numpy(x[:, start : start + 4]), dim=-1).numpy()
        assert np.allclose(out[:, start : start + 4], part, atol=1e-6)


@pytest.mark.parametrize("is_causal", (False, True))
@pytest.mark.parametrize("seq_len", (80, 1))
def test_attention_against_torch(seq_len, is_causal):
    # reference: tests/test_attention.py:99-117 (fp16: rtol = atol = 0.01, scale 1)
    q, k, v = (_half(2, 2, seq_len, 32) for _ in range(3))
    out = oracle.attention(q.numpy(), k.numpy(), v.numpy(), is_causal=is_causal, bm=32, bn=16)
    expected = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=is_causal, scale=1).numpy()
    assert np.allclose(out, expected, rtol=0.01, atol=0.01)


def test_attention_closed_forms():
    q, v = _half(1, 1, 20, 16), _half(1, 1, 20, 16)
    k = torch.zeros(1, 1, 20, 16, dtype=torch.float16)
    out = oracle.attention(q.numpy(), k.numpy(), v.numpy(), bm=8, bn=8)
    mean = v.float().mean(dim=2, keepdim=True).numpy()
    assert np.allclose(out, np.broadcast_to(mean, out.shape), atol=2e-3)  # identical keys -> mean of V
    causal = oracle.attention(q.numpy(), k.numpy(), v.numpy(), is_causal=True, bm=8, bn=8)
    assert np.allclose(causal[0, 0, 0], v.float().numpy()[0, 0, 0], atol=1e-3)  # row 0 sees only key 0
    prefix_mean = v.float().numpy()[0, 0, :5].mean(axis=0)
    assert np.allclose(causal[0, 0, 4], prefix_mean, atol=2e-3)  # row 4 sees keys 0..4
    scaled = oracle.attention(q.numpy(), q.numpy(), v.numpy(), scale=0.25, bm=8, bn=8)
    expected = F.scaled_dot_product_attention(q.float(), q.float(), v.float(), scale=0.25).numpy()
    assert np.allclose(scaled, expected, rtol=0.01, atol=0.01)


@pytest.mark.parametrize("padding", (0, (1, 1), (0, 1), (2, 0)))
def test_conv2d_against_torch(padding):
    # reference: tests/test_conv2d.py:116-133 (torch.rand inputs, rtol = atol = 1e-3 in fp16 there;
    # here the comparison is against the fp32 conv of the same fp16 values, rounded once)
    x = torch.rand(2, 6, 9, 8).to(torch.float16)
    w = torch.rand(5, 6, 3, 3).to(torch.float16)
    pad = (padding, padding) if isinstance(padding, int) else padding
    out = oracle.conv2d(x.numpy(), w.numpy(), padding=pad, bm=16, bn=4, bk=8)
    expected = F.conv2d(x.float(), w.float(), padding=pad).to(torch.float16).float().numpy()
    assert out.shape == expected.shape
    assert np.allclose(out, expected, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("stride, dilation, padding", (((2, 2), (1, 1), (1, 1)), ((1, 2), (2, 1), (0, 1)), ((3, 1), (1, 2), (2, 2)), ((2, 3), (2, 2), (2, 0))))
def test_conv2d_with_stride_and_dilation_against_torch(stride, dilation, padding):
    """`tile(..., strides, dilation)` of the arrangement (reference src/ninetoothed/tensor.py:199-286): with
    `floor_mode` the windows are those of `F.conv2d`; without it `tile` rounds the count up, and the extra
    window equals what `F.conv2d` computes on an input that is zero-padded further at the bottom / right."""
    x = torch.rand(2, 5, 11, 10).to(torch.float16)
    w = torch.rand(4, 5, 3, 2).to(torch.float16)
    out = oracle.conv2d(x.numpy(), w.numpy(), padding=padding, bm=16, bn=4, bk=8, stride=stride, dilation=dilation, floor_mode=True)
    expected = F.conv2d(x.float(), w.float(), padding=padding, stride=stride, dilation=dilation).to(torch.float16).float().numpy()
    assert out.shape == expected.shape
    assert np.allclose(out, expected, rtol=1e-3, atol=1e-3)
    hanging = oracle.conv2d(x.numpy(), w.numpy(), padding=padding, bm=16, bn=4, bk=8, stride=stride, dilation=dilation, floor_mode=False)
    padded = F.pad(x.float(), (padding[1], padding[1] + stride[1], padding[0], padding[0] + stride[0]))
    wider = F.conv2d(padded, w.float(), stride=stride, dilation=dilation).to(torch.float16).float().numpy()
    assert hanging.shape[2] in (out.shape[2], out.shape[2] + 1) and hanging.shape[3] in (out.shape[3], out.shape[3] + 1)
    assert np.allclose(hanging, wider[:, :, : hanging.shape[2], : hanging.shape[3]], rtol=1e-3, atol=1e-3)


def test_conv2d_1x1_is_matmul():
    x = _half(2, 8, 4, 4)
    w = _half(6, 8, 1, 1)
    out = oracle.conv2d(x.numpy(), w.numpy(), bm=8, bn=2, bk=4)
    a = x.float().permute(0, 2, 3, 1).reshape(-1, 8)
    expected = (a @ w.float().reshape(6, 8).T).to(torch.float16).float().reshape(2, 4, 4, 6).permute(0, 3, 1, 2).numpy()
    assert np.allclose(out, expected, rtol=1e-3, atol=1e-3)


# ---- what Triton itself computes (vectors written by tests/golden/make_triton_*_vectors.py) ----


def _golden(name):
    import json
    import pathlib

    return json.loads((pathlib.Path(__file__).resolve().parent / "golden" / name).read_text())


def test_triton_rand_matches_the_vectors_of_the_installed_triton():
    """``tl.rand`` outputs for int32 and int64 offsets (up to 2^62) and seeds up to 2^62: pins the
    output word, the placement of the offset's and the seed's halves, the mirroring and the scale."""
    cases = _golden("triton_rand_vectors.json")["cases"]
    assert len(cases) >= 18
    for case in cases:
        got = oracle.triton_rand(case["seed"], np.array(case["offsets"], dtype=np.int64))
        assert np.array_equal(got.view(np.int32), np.array(case["bits"], dtype=np.int32)), (case["seed"], case["offset_dtype"])


def test_rounding_points_match_the_vectors_of_the_installed_triton():
    """A tile times a Python literal is computed in the tile's type with the literal rounded to it
    first; a tile times a run-time scalar in fp32; the addmm epilogue in fp32 on the rounded product."""
    cases = _golden("triton_promotion_vectors.json")["cases"]

    def half(bits):
        return np.array(bits, dtype=np.int16).view(np.float16).astype(np.float32)

    literal = cases["literal_fp16"]
    factor = oracle._round(np.float32(oracle.LOG2E), "fp16").astype(np.float32)
    assert float(factor) == 1.4423828125
    got = oracle._round(half(literal["q"]) * factor, "fp16")
    assert np.array_equal(got.view(np.int16), np.array(literal["out"], dtype=np.int16))
    unrounded = oracle._round(half(literal["q"]) * np.float32(oracle.LOG2E), "fp16")
    assert not np.array_equal(unrounded.view(np.int16), np.array(literal["out"], dtype=np.int16))  # the vectors tell the two apart

    scaled = cases["scaled_fp16"]
    factor = np.float32(scaled["scale"]) * np.float32(oracle.LOG2E)
    got = oracle._round(half(scaled["q"]) * factor, "fp16")
    assert np.array_equal(got.view(np.int16), np.array(scaled["out"], dtype=np.int16))

    # the same two rules through the attention restatement itself: one key, so the output is V whatever Q is,
    # and the factor is visible through a two-key problem solved in closed form below
    epilogue = cases["addmm_epilogue_fp16"]
    product = np.array(epilogue["product"], dtype=np.int32).view(np.float32)
    n = product.size
    # addmm with K = 1: mat1 = product rounded apart into two fp16 factors is not exact, so check the epilogue rule
    # on the restatement's own arithmetic: beta * input + alpha * round16(product), in fp32, rounded once
    rounded = product.astype(np.float16).astype(np.float32)
    got = (np.float32(epilogue["beta"]) * half(epilogue["input"]) + np.float32(epilogue["alpha"]) * rounded).astype(np.float16)
    assert np.array_equal(got.view(np.int16), np.array(epilogue["out"], dtype=np.int16))
    # and the restatement does exactly that: a 1 x n problem whose product is exact in fp16 (powers of two)
    input = half(epilogue["input"]).astype(np.float16).reshape(1, n)
    mat1 = np.array([[2.0]], dtype=np.float16)
    mat2 = np.ldexp(1.0, np.arange(n) % 11 - 5).astype(np.float16).reshape(1, n)
    out = oracle.addmm(input, mat1, mat2, epilogue["beta"], epilogue["alpha"], bm=1, bn=64, bk=1)
    expected = (np.float32(epilogue["beta"]) * input.astype(np.float32) + np.float32(epilogue["alpha"]) * (2.0 * mat2.astype(np.float32))).astype(np.float16)
    assert np.array_equal(out.astype(np.float16).view(np.int16), expected.view(np.int16))


def test_attention_literal_factor_is_rounded_to_the_tile_type():
    """Two keys, one query, head dimension 1: the output weight of key 0 is 1 / (1 + 2^(q' (k1 - k0))) with
    q' = round16(q * 1.4423828125) for the reference program and round16(q * fp32(scale * log2 e)) with a scale."""
    candidates = np.arange(4.0, 8.0, 2.0**-8, dtype=np.float32).astype(np.float16)  # every half in [4, 8)
    differ = np.float16(candidates.astype(np.float32) * np.float32(1.4423828125)) != np.float16(candidates.astype(np.float32) * np.float32(oracle.LOG2E))
    q = candidates[np.nonzero(differ)[0][:1]].reshape(1, 1, 1, 1)  # the two factors round this one to different halves
    k = np.array([[[[0.0], [1.0]]]], dtype=np.float16)
    v = np.array([[[[1.0], [0.0]]]], dtype=np.float16)
    literal = np.float16(np.float32(q[0, 0, 0, 0]) * np.float32(1.4423828125))
    full = np.float16(np.float32(q[0, 0, 0, 0]) * np.float32(oracle.LOG2E))
    assert literal != full
    out = oracle.attention(q, k, v, bm=1, bn=2)
    assert np.isclose(out[0, 0, 0, 0], 1.0 / (1.0 + 2.0 ** float(literal)), rtol=1e-3)
    assert not np.isclose(out[0, 0, 0, 0], 1.0 / (1.0 + 2.0 ** float(full)), rtol=1e-3)
    scaled = oracle.attention(q, k, v, scale=1.0, bm=1, bn=2)
    assert np.isclose(scaled[0, 0, 0, 0], 1.0 / (1.0 + 2.0 ** float(full)), rtol=1e-3)
