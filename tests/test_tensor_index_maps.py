"""The product's symbolic front-end (Tensor / Symbol / eval / subs) against
the reference's golden vectors and against the brute-force oracle."""

import numpy as np
import pytest

import ninetoothed_amd as ninetoothed
from ninetoothed_amd import Symbol, Tensor, programs
from oracle import programs as oracle_programs
from oracle.arrangement import View
from tests.golden_vectors import load


@pytest.mark.parametrize("shape_options", (None, {"constexpr": True}))
@pytest.mark.parametrize("subs_before_eval", (False, True))
@pytest.mark.parametrize("use_tensor_in_subs", (False, True))
def test_eval(use_tensor_in_subs, subs_before_eval, shape_options):
    # same scenario as the reference's tests/test_eval.py:8-198
    g = load("eval_vectors.json")
    assert np.array_equal(Tensor(shape=(2, 3)).eval(), g[0])

    x = Tensor(2, shape_options=shape_options)
    block_size_m = ninetoothed.block_size()
    block_size_n = ninetoothed.block_size()
    subs = {x: {"shape": (5, 6)}, block_size_m: 2, block_size_n: 3}
    if use_tensor_in_subs:
        subs[x] = Tensor(shape=subs[x]["shape"])

    def evaluated(tensor):
        return tensor.subs(subs).eval() if subs_before_eval else tensor.eval(subs)

    assert np.array_equal(evaluated(x), g[1])
    assert np.array_equal(evaluated(x.permute((1, 0))), g[2])
    x_tiled = x.tile((block_size_m, block_size_n))
    assert np.array_equal(evaluated(x_tiled), g[3])
    x_tiled_tiled = x_tiled.tile((block_size_m, block_size_n))
    assert np.array_equal(evaluated(x_tiled_tiled), g[4])
    x_tiled_tiled.dtype = x_tiled_tiled.dtype.flatten()
    assert np.array_equal(evaluated(x_tiled_tiled), g[5])
    x_tiled_tiled.dtype.dtype = x_tiled_tiled.dtype.dtype.flatten()
    assert np.array_equal(evaluated(x_tiled_tiled), g[6])


def test_unsqueeze():
    # reference: tests/test_unsqueeze.py:7-58
    g = load("unsqueeze_vectors.json")
    x = Tensor(1)
    block_size_m = ninetoothed.block_size()
    block_size_n = ninetoothed.block_size()
    subs = {x: {"shape": (5,)}, block_size_m: 2, block_size_n: 3}
    x_unsqueezed = x.unsqueeze(0)
    assert np.array_equal(x_unsqueezed.eval(subs), g[0])
    x_unsqueezed_expanded = x_unsqueezed.expand((3, -1))
    assert np.array_equal(x_unsqueezed_expanded.eval(subs), g[1])
    assert np.array_equal(x_unsqueezed_expanded.tile((block_size_m, block_size_n)).eval(subs), g[2])
    x_tiled_unsqueezed = x.tile((block_size_n,)).unsqueeze(0)
    assert np.array_equal(x_tiled_unsqueezed.eval(subs), g[3])
    assert np.array_equal(x_tiled_unsqueezed.expand((3, -1)).eval(subs), g[4])


@pytest.mark.parametrize(
    "shape, indices",
    (
        ((3, 4, 2), slice(None, None, None)),
        ((3, 4, 2), slice(0, -1, 2)),
        ((2, 3, 4, 5), slice(1, None, 2)),
        ((3, 4, 2), (slice(None), 1, slice(None))),
        ((3, 4, 2), (1, slice(None), None)),
        ((3, 4, 2), (slice(None, None, -1), 0, slice(1, -1))),
        ((3, 4, 2), (..., 1)),
        ((3, 4, 2), (None, slice(None), 1, slice(None))),
        ((6, 5), (slice(2, 4, None), slice(1, 4, None))),
    ),
)
def test_getitem(shape, indices):
    # reference: tests/test_getitem.py:7-32
    output = Tensor(shape=shape)[indices].eval()
    expected = np.arange(np.prod(shape)).reshape(shape)[indices]
    assert output.shape == expected.shape and np.array_equal(output, expected)


def test_addmm_arrangement():
    # reference: tests/test_debugging.py:249-256 (CPU half of that test)
    import functools

    g = load("debugging_vectors.json")
    targets = g[6:]
    arrangement = functools.partial(programs.addmm.arrangement, BLOCK_SIZE_M=2, BLOCK_SIZE_N=2, BLOCK_SIZE_K=2)
    tensors = (Tensor(shape=(3, 4)), Tensor(shape=(3, 5)), Tensor(shape=(5, 4)), Tensor(0), Tensor(0), Tensor(shape=(3, 4)))
    for arranged, expected in zip(arrangement(*tensors), targets):
        result = arranged.flatten().eval() if arranged.ndim != 0 else arranged.eval()
        assert np.array_equal(result, expected)


def test_meta_operations_do_not_touch_their_input():
    x = Tensor(2)
    shape = x.shape
    x.tile((2, 2)).expand((-1, -1))
    assert x.shape == shape and x.source is x and not isinstance(x.dtype, Tensor)


def test_symbol_folding_and_flags():
    s = Symbol("BLOCK", meta=True)
    assert s.lower_bound == 32 and s.upper_bound == 1024 and s.power_of_two
    c = Symbol("N", constexpr=True)
    assert c.lower_bound == 1 and c.upper_bound == 2**20 and not c.power_of_two
    assert (s + 0) == s and (s * 1) == s and (s // 1) == s and (0 + s) == s
    assert ((s + 3) * 2).evaluate({"BLOCK": 5}) == 16
    assert Symbol(4) == 4 and Symbol(4) != 5
    with pytest.raises(ValueError):
        Symbol(3, constexpr=True)
    b = ninetoothed.block_size(lower_bound=64, upper_bound=128)
    assert b.meta and b.lower_bound == 64 and b.upper_bound == 128


@pytest.mark.parametrize("m, n, k, bm, bn, bk", ((3, 4, 5, 2, 2, 2), (17, 9, 20, 4, 8, 16), (8, 8, 8, 8, 8, 8)))
def test_matmul_arrangement_matches_oracle(m, n, k, bm, bn, bk):
    lhs, rhs, out = programs.matmul.arrangement(Tensor(shape=(m, k)), Tensor(shape=(k, n)), Tensor(shape=(m, n)), bm, bn, bk)
    o_lhs, o_rhs, o_out = oracle_programs.arrange_matmul(View.of_shape((m, k)), View.of_shape((k, n)), View.of_shape((m, n)), bm, bn, bk)
    assert np.array_equal(lhs.eval(), o_lhs.table)
    assert np.array_equal(rhs.eval(), o_rhs.table)
    assert np.array_equal(out.eval(), o_out.table)


@pytest.mark.parametrize("padding", ((0, 0), (1, 1), (0, 1), (2, 0)))
def test_conv2d_arrangement_matches_oracle_and_unfold(padding):
    import torch
    import torch.nn.functional as F

    n, c, h, w, k, r, s = 2, 3, 6, 5, 4, 3, 2
    p, q = h + 2 * padding[0] - r + 1, w + 2 * padding[1] - s + 1
    x_t, w_t, y_t = Tensor(shape=(n, c, h, w)), Tensor(shape=(k, c, r, s)), Tensor(shape=(n, k, p, q))
    lhs, rhs, out = programs.conv2d.arrangement(x_t, w_t, y_t, BLOCK_SIZE_M=4, BLOCK_SIZE_N=2, BLOCK_SIZE_K=8)
    subs = {Symbol("padding_h", constexpr=True): padding[0], Symbol("padding_w", constexpr=True): padding[1]}

    x_view = View.of_shape((n, c, h, w)).pad(((0, 0), (0, 0), (padding[0],) * 2, (padding[1],) * 2))
    x_view = x_view.tile((1, c, r, s), strides=(-1, -1, 1, 1)).squeeze(1).squeeze(0, level=1).ravel().flatten(end_dim=3).flatten(start_dim=1)
    w_view = View.of_shape((k, c, r, s)).flatten(start_dim=1).permute((1, 0))
    y_view = View.of_shape((n, k, p, q)).permute((0, 2, 3, 1)).flatten(end_dim=3)
    o_lhs, o_rhs, o_out = oracle_programs.arrange_matmul(x_view, w_view, y_view, 4, 2, 8)
    assert np.array_equal(lhs.eval(subs), o_lhs.table)
    assert np.array_equal(rhs.eval(subs), o_rhs.table)
    assert np.array_equal(out.eval(subs), o_out.table)

    # closed form: the A view is im2col, i.e. torch's unfold with (c, r, s) ordering
    values = torch.arange(n * c * h * w, dtype=torch.float32).reshape(n, c, h, w) + 1
    columns = F.unfold(values, (r, s), padding=padding)  # [n, c*r*s, p*q]
    im2col = columns.permute(0, 2, 1).reshape(n * p * q, c * r * s).numpy()
    mine = np.where(x_view.table >= 0, x_view.table + 1, 0)
    assert np.array_equal(mine, im2col)


def test_simulate_arrangement_matches_the_reference_vectors():
    # reference: tests/test_debugging.py:12-239 (addmm arrangement, m=3, n=4, k=5, 2x2x2 blocks):
    # six source tensors followed by six target tensors
    import functools

    from ninetoothed_amd import programs
    from ninetoothed_amd.debugging import simulate_arrangement
    from tests.golden_vectors import load

    vectors = load("debugging_vectors.json")
    arrangement = functools.partial(programs.addmm.arrangement, BLOCK_SIZE_M=2, BLOCK_SIZE_N=2, BLOCK_SIZE_K=2)
    tensors = (Tensor(shape=(3, 4)), Tensor(shape=(3, 5)), Tensor(shape=(5, 4)), Tensor(0), Tensor(0), Tensor(shape=(3, 4)))
    sources, targets = simulate_arrangement(arrangement, tensors, device="cpu")
    assert len(sources) == len(targets) == 6
    for position in range(6):
        assert np.array_equal(sources[position].numpy(), vectors[position]), position
        assert np.array_equal(targets[position].numpy(), vectors[6 + position]), position


def test_naming_prefixes_as_the_reference_spells_them():
    """``ninetoothed.naming`` (reference tests/test_naming.py:4-49): the strings of the three kinds of prefix, that
    they stack, that a meta name counts as a constant, and that removing them gives back the bare name -- also one
    that itself starts with ``ninetoothed_``."""
    import ninetoothed.naming as by_reference_name

    from ninetoothed_amd import naming

    assert by_reference_name is naming
    name = "ninetoothed_name"
    assert naming.make_constexpr(name) == "ninetoothed_constexpr_prefix_ninetoothed_name"
    assert naming.make_meta(name) == "ninetoothed_meta_prefix_ninetoothed_name"
    assert naming.make_next_power_of_2(name) == "ninetoothed_next_power_of_2_prefix_ninetoothed_name"
    stacked = naming.make_next_power_of_2(naming.make_constexpr(name))
    assert stacked == "ninetoothed_next_power_of_2_prefix_ninetoothed_constexpr_prefix_ninetoothed_name"
    assert naming.is_constexpr(naming.make_constexpr(name)) and naming.is_constexpr(naming.make_meta(name)) and naming.is_constexpr(stacked)
    assert naming.is_meta(naming.make_meta(name)) and not naming.is_meta(naming.make_constexpr(name))
    assert naming.is_next_power_of_2(naming.make_next_power_of_2(name)) and naming.is_next_power_of_2(stacked)
    assert not naming.is_constexpr(name) and not naming.is_meta(name) and not naming.is_next_power_of_2(name)
    for mangled in (naming.make_constexpr(name), naming.make_meta(name), naming.make_next_power_of_2(name), stacked):
        assert naming.remove_prefixes(mangled) == name
    assert naming.remove_prefixes("x") == "x"
    assert naming.auto_generate("libdevice") == "ninetoothed_libdevice"


def test_submodules_that_share_a_name_with_a_public_function():
    """``jit`` and ``eval`` are submodules and public functions at once in the reference
    (src/ninetoothed/__init__.py:16-18); importing the submodule must not replace the function, under either
    package name.  ``generation.CACHE_DIR`` and ``utils.calculate_default_configs`` are what the reference's
    own tests and ``jit`` reach for in those modules (tests/test_aot.py:37, src/ninetoothed/jit.py:55-57)."""
    import importlib
    import pathlib

    import ninetoothed
    import ninetoothed.generation
    import ninetoothed.utils
    import ninetoothed_amd
    from ninetoothed.eval import _eval, _subs
    from ninetoothed.jit import jit

    jit_module = importlib.import_module("ninetoothed.jit")
    assert jit_module is importlib.import_module("ninetoothed_amd.jit")
    assert jit is ninetoothed.jit is ninetoothed_amd.jit is jit_module.jit and callable(jit)
    assert _eval is ninetoothed.eval is ninetoothed_amd.eval and _subs is ninetoothed.subs
    assert isinstance(ninetoothed.generation.CACHE_DIR, pathlib.Path)
    assert ninetoothed.utils.calculate_default_configs() == (8, 5)
    x = ninetoothed.Tensor(shape=(4, 6))
    assert ninetoothed.eval(x.tile((2, 3))).shape == (2, 2, 2, 3)
