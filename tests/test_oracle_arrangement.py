"""Pins the CPU oracle for index maps (oracle/arrangement.py) against the
vectors the reference's own tests hold, and against closed forms."""

import numpy as np
import pytest

from oracle.arrangement import View
from tests.golden_vectors import load


def test_eval_vectors():
    # reference: tests/test_eval.py:12-198 (5x6 tensor, blocks 2x3)
    g = load("eval_vectors.json")
    assert np.array_equal(View.of_shape((2, 3)).table, g[0])
    x = View.of_shape((5, 6))
    assert np.array_equal(x.table, g[1])
    assert np.array_equal(x.permute((1, 0)).table, g[2])
    tiled = x.tile((2, 3))
    assert np.array_equal(tiled.table, g[3])
    tiled_tiled = tiled.tile((2, 3))
    assert np.array_equal(tiled_tiled.table, g[4])
    inner_flat = tiled_tiled.flatten(level=1)
    assert np.array_equal(inner_flat.table, g[5])
    assert np.array_equal(inner_flat.flatten(level=2).table, g[6])


def test_unsqueeze_vectors():
    # reference: tests/test_unsqueeze.py:17-58
    g = load("unsqueeze_vectors.json")
    x = View.of_shape((5,))
    unsqueezed = x.unsqueeze(0)
    assert np.array_equal(unsqueezed.table, g[0])
    expanded = unsqueezed.expand((3, -1))
    assert np.array_equal(expanded.table, g[1])
    assert np.array_equal(expanded.tile((2, 3)).table, g[2])
    tiled_unsqueezed = x.tile((3,)).unsqueeze(0)
    assert np.array_equal(tiled_unsqueezed.table, g[3])
    assert np.array_equal(tiled_unsqueezed.expand((3, -1)).table, g[4])


def _matmul_views(m, n, k, bm, bn, bk):
    from oracle.programs import arrange_matmul

    return arrange_matmul(View.of_shape((m, k)), View.of_shape((k, n)), View.of_shape((m, n)), bm, bn, bk)


def test_addmm_arrangement_vectors():
    # reference: tests/test_debugging.py:41-239 -- per-program views of the addmm
    # arrangement for m=3, n=4, k=5 with 2x2x2 blocks; the grid level is flattened
    g = load("debugging_vectors.json")
    targets = g[6:]
    lhs, rhs, out = _matmul_views(3, 4, 5, 2, 2, 2)
    input_view = View.of_shape((3, 4)).tile((2, 2))
    assert np.array_equal(input_view.flatten().table, targets[0])
    assert np.array_equal(lhs.flatten().table, targets[1])
    assert np.array_equal(rhs.flatten().table, targets[2])
    assert np.array_equal(out.flatten().table, targets[5])


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
def test_getitem_is_numpy_indexing(shape, indices):
    # reference: tests/test_getitem.py:25-32 (closed form: basic indexing of arange)
    expected = np.arange(np.prod(shape)).reshape(shape)[indices]
    assert np.array_equal(View.of_shape(shape).getitem(indices).table, expected)


def test_unit_stride_tiles_are_sliding_windows():
    # closed form: tile(strides=1) == numpy's sliding_window_view
    x = View.of_shape((7, 9))
    tiled = x.tile((3, 4), strides=(1, 1))
    windows = np.lib.stride_tricks.sliding_window_view(np.arange(63).reshape(7, 9), (3, 4))
    assert np.array_equal(tiled.table, windows)


def test_tile_with_dilation_and_padding_masks():
    x = View.of_shape((6,)).pad(((2, 1),))
    assert np.array_equal(x.table, [-1, -1, 0, 1, 2, 3, 4, 5, -1])
    tiled = x.tile((2,), strides=(3,), dilation=(2,))
    # outer = ceil((9 - 2*(2-1) - 1) / 3) + 1 = 3 tiles at 0, 3, 6 with elements {o, o+2}
    assert np.array_equal(tiled.table, [[-1, 0], [1, 3], [4, -1]])
