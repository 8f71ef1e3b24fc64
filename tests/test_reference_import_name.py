"""Programs that start with the reference's own import lines
(``import ninetoothed``, ``import ninetoothed.language as ntl``,
``from ninetoothed import Tensor``; README.md:30-34 and the head of every
program under the reference's tests/) run on this build: the five programs are
written out here against that name and checked against the CPU oracle and the
torch operator the reference's tests compare with (tests/test_matmul.py:86-88,
tests/test_addmm.py:88-90, tests/test_softmax.py:38-40,
tests/test_attention.py:115-117, tests/test_conv2d.py:131-133)."""

import functools

import ninetoothed
import ninetoothed.language as ntl
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from ninetoothed import Symbol, Tensor, block_size

from oracle import programs as oracle

HALF_TOL = dict(rtol=1e-2, atol=1e-2)


def test_the_name_is_an_alias_not_a_copy():
    import ninetoothed_amd
    import ninetoothed_amd.auto_tuner
    import ninetoothed_amd.debugging
    import ninetoothed_amd.language

    assert ntl is ninetoothed_amd.language
    assert Tensor is ninetoothed_amd.Tensor and Symbol is ninetoothed_amd.Symbol
    assert ninetoothed.make is ninetoothed_amd.make and ninetoothed.jit is ninetoothed_amd.jit
    from ninetoothed.auto_tuner import AutoTuner
    from ninetoothed.debugging import simulate_arrangement
    from ninetoothed.language import libdevice

    assert AutoTuner is ninetoothed_amd.auto_tuner.AutoTuner
    assert simulate_arrangement is ninetoothed_amd.debugging.simulate_arrangement
    assert libdevice is ninetoothed_amd.language.libdevice
    assert set(ninetoothed.__all__) >= {"Symbol", "Tensor", "block_size", "build", "eval", "subs", "jit", "make", "float16", "bfloat16", "float32"}
    with pytest.raises(ModuleNotFoundError):
        __import__("ninetoothed.no_such_module")


# ---- the five programs, written against `ninetoothed` ----------------------

TILE_M = block_size()
TILE_N = block_size()
TILE_K = block_size()


def product_arrangement(left, right, result, tile_m=TILE_M, tile_n=TILE_N, tile_k=TILE_K):
    result_tiles = result.tile((tile_m, tile_n))

    left_tiles = left.tile((tile_m, tile_k)).tile((1, -1))
    left_tiles = left_tiles.expand((-1, result_tiles.shape[1]))
    left_tiles.dtype = left_tiles.dtype.squeeze(0)

    right_tiles = right.tile((tile_k, tile_n)).tile((-1, 1))
    right_tiles = right_tiles.expand((result_tiles.shape[0], -1))
    right_tiles.dtype = right_tiles.dtype.squeeze(1)

    return left_tiles, right_tiles, result_tiles


def product_application(left, right, result):
    total = ntl.zeros(result.shape, dtype=ntl.float32)
    for step in range(left.shape[0]):
        total += ntl.dot(left[step], right[step])
    result = total.to(ntl.float16)  # noqa: F841


def addmm_arrangement(bias, left, right, beta, alpha, result):
    _, _, bias_tiles = product_arrangement(left, right, bias)
    left_tiles, right_tiles, result_tiles = product_arrangement(left, right, result)
    return bias_tiles, left_tiles, right_tiles, beta, alpha, result_tiles


def addmm_application(bias, left, right, beta, alpha, result):
    product = ntl.zeros(result.shape, dtype=ntl.float32)
    product_application(left, right, product)
    result = beta * bias + alpha * product  # noqa: F841


ROW_LENGTH = Symbol("ROW_LENGTH", constexpr=True)


@ninetoothed.jit
def softmax_kernel(
    source_row: Tensor(2, other=float("-inf")).tile((1, ROW_LENGTH)),
    target_row: Tensor(2).tile((1, ROW_LENGTH)),
):
    shifted = source_row - ntl.max(source_row)
    weights = ntl.exp(shifted)
    target_row = weights / ntl.sum(weights)  # noqa: F841


QUERY_ROWS = block_size(lower_bound=64, upper_bound=128)
KEY_ROWS = block_size(lower_bound=32, upper_bound=64)


def attention_arrangement(q, k, v, is_causal, o, query_rows=QUERY_ROWS, key_rows=KEY_ROWS):
    def per_query_block(tensor):
        blocks = tensor.tile((1, 1, query_rows, -1))
        blocks.dtype = blocks.dtype.squeeze((0, 1))
        return blocks

    q_blocks = per_query_block(q)

    def all_key_blocks(tensor):
        blocks = tensor.tile((1, 1, key_rows, -1)).tile((1, 1, -1, -1))
        blocks = blocks.expand((-1, -1, q_blocks.shape[-2], -1))
        blocks.dtype = blocks.dtype.squeeze((0, 1, 3))
        blocks.dtype.dtype = blocks.dtype.dtype.squeeze((0, 1))
        return blocks

    return q_blocks, all_key_blocks(k), all_key_blocks(v), is_causal, per_query_block(o)


def attention_application(q, k, v, is_causal, o):
    queries = (q * 1.44269504089).to(q.dtype)
    out = ntl.zeros((q.shape[-2], q.shape[-1]), dtype=ntl.float32)
    denominator = ntl.full((q.shape[-2],), 1, dtype=ntl.float32)
    highest = ntl.full((q.shape[-2],), float("-inf"), dtype=ntl.float32)
    for j in range(k.shape[0]):
        scores = ntl.dot(queries, ntl.trans(k[j]))
        scores = ntl.where(k[j].offsets(-2) < k.source.shape[-2], scores, float("-inf"))
        if is_causal:
            visible = q.offsets(-2)[:, None] >= k[j].offsets(-2)[None, :]
            scores = ntl.where(visible, scores, float("-inf"))
        new_highest = ntl.maximum(highest, ntl.max(scores, 1))
        weights = ntl.exp2(scores - new_highest[:, None])
        shrink = ntl.exp2(highest - new_highest)
        out = out * shrink[:, None] + ntl.dot(weights.to(v[j].dtype), v[j])
        denominator = denominator * shrink + ntl.sum(weights, 1)
        highest = new_highest
    out /= denominator[:, None]
    o = out  # noqa: F841


def conv2d_arrangement(image, filters, result):
    pad_h = Symbol("padding_h", constexpr=True)
    pad_w = Symbol("padding_w", constexpr=True)
    image = image.pad(((0, 0), (0, 0), (pad_h, pad_h), (pad_w, pad_w)))
    windows = image.tile((1, *filters.shape[1:]), strides=(-1, -1, 1, 1)).squeeze(1)
    windows.dtype = windows.dtype.squeeze(0)
    rows = windows.ravel().flatten(end_dim=3).flatten(start_dim=1)
    columns = filters.flatten(start_dim=1).permute((1, 0))
    pixels = result.permute((0, 2, 3, 1)).flatten(end_dim=3)
    return product_arrangement(rows, columns, pixels)


# ---- on the GPU ----------------------------------------------------------------


def _half(*shape, scale=1.0):
    return (torch.randn(*shape) * scale).to(torch.float16)


@pytest.mark.gpu
def test_matmul_program():
    a, b = _half(192, 160), _half(160, 224)
    kernel = ninetoothed.make(product_arrangement, product_application, (Tensor(2), Tensor(2), Tensor(2)))
    out = torch.empty(192, 224, dtype=torch.float16, device="cuda")
    kernel(a.cuda(), b.cuda(), out)
    assert kernel.last_plan.startswith("launch_nt_matmul")
    assert np.allclose(out.cpu().float().numpy(), oracle.matmul(a.numpy(), b.numpy(), 64, 64, 64), **HALF_TOL)
    assert torch.allclose(out, torch.matmul(a.cuda(), b.cuda()), **HALF_TOL)


@pytest.mark.gpu
def test_addmm_program():
    bias, a, b = _half(130, 72), _half(130, 96), _half(96, 72)
    kernel = ninetoothed.make(addmm_arrangement, addmm_application, (Tensor(2), Tensor(2), Tensor(2), Tensor(0), Tensor(0), Tensor(2)))
    out = torch.empty(130, 72, dtype=torch.float16, device="cuda")
    kernel(bias.cuda(), a.cuda(), b.cuda(), 0.5, 1.25, out)
    assert kernel.last_plan.startswith("launch_nt_addmm")
    expected = oracle.addmm(bias.numpy(), a.numpy(), b.numpy(), 0.5, 1.25)
    assert np.allclose(out.cpu().float().numpy(), expected, **HALF_TOL)
    assert torch.allclose(out, torch.addmm(bias.cuda(), a.cuda(), b.cuda(), beta=0.5, alpha=1.25), rtol=1e-2, atol=0.075)


@pytest.mark.gpu
def test_softmax_program():
    x = torch.randn(37, 781)
    y = torch.empty_like(x, device="cuda")
    softmax_kernel(x.cuda(), y, ROW_LENGTH=781)
    assert softmax_kernel.last_plan.startswith("launch_nt_softmax")
    assert np.allclose(y.cpu().numpy(), oracle.softmax(x.numpy()), rtol=1e-5, atol=1e-6)
    assert torch.allclose(y, torch.softmax(x.cuda(), dim=-1), rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("is_causal", (False, True))
def test_attention_program(is_causal):
    q, k, v = (_half(2, 3, 200, 64) for _ in range(3))
    options = (None, None, {"constexpr": True}, {"constexpr": True, "upper_bound": 128})
    tensors = tuple(Tensor(4, shape_options=options) for _ in range(3)) + (Tensor(0, constexpr=True), Tensor(4, shape_options=options))
    kernel = ninetoothed.make(attention_arrangement, attention_application, tensors)
    o = torch.empty_like(q, device="cuda")
    kernel(q.cuda(), k.cuda(), v.cuda(), is_causal, o)
    assert kernel.last_plan.startswith("launch_nt_attention")
    expected = oracle.attention(q.numpy(), k.numpy(), v.numpy(), is_causal=is_causal)
    assert np.allclose(o.cpu().float().numpy(), expected, **HALF_TOL)
    assert torch.allclose(o, F.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=is_causal, scale=1), **HALF_TOL)


@pytest.mark.gpu
def test_conv2d_program():
    x, w = _half(3, 16, 12, 11, scale=0.3), _half(24, 16, 3, 3, scale=0.3)
    kernel = ninetoothed.make(conv2d_arrangement, product_application, (Tensor(4), Tensor(4, shape_options={"constexpr": True}), Tensor(4)), max_num_configs=50)
    y = torch.empty(3, 24, 12, 11, dtype=torch.float16, device="cuda")
    kernel(x.cuda(), w.cuda(), y, padding_h=1, padding_w=1)
    assert kernel.last_plan.startswith("launch_nt_conv2d")
    expected = oracle.conv2d(x.numpy(), w.numpy(), padding=(1, 1), bm=32, bn=32, bk=32)
    assert np.allclose(y.cpu().float().numpy(), expected, **HALF_TOL)
    assert torch.allclose(y, F.conv2d(x.cuda(), w.cuda(), padding=1), **HALF_TOL)


@pytest.mark.gpu
def test_readme_style_program_with_functools_partial():
    """Fixed block sizes bound with ``functools.partial``, as the reference's tests bind them."""
    arrangement = functools.partial(product_arrangement, tile_m=64, tile_n=64, tile_k=64)
    kernel = ninetoothed.make(arrangement, product_application, (Tensor(2), Tensor(2), Tensor(2)))
    a, b = _half(512, 512), _half(512, 512)
    out = torch.empty(512, 512, dtype=torch.float16, device="cuda")
    kernel(a.cuda(), b.cuda(), out)
    assert torch.allclose(out, torch.matmul(a.cuda(), b.cuda()), **HALF_TOL)
