"""TEST INFRASTRUCTURE ONLY -- CPU oracle for arrangements (index maps).

Nothing in the product imports this module; only ``tests/``, the smoke check
and the CPU-baseline leg of ``bench.py`` do.

A :class:`View` restates what an arranged tensor of the reference *means* by
brute force: it holds, for every position of every level, the flat offset of
the source element that position refers to (row-major source), or ``-1`` where
the position is masked.  Meta-operations are array manipulations on that table,
so there is no symbolic algebra to get wrong:

* ``tile``    -- reference src/ninetoothed/tensor.py:199-286 (outer size
  ``ceil((size - dilation*(tile-1) - 1) / stride) + 1``; element ``(o, t)`` is
  source index ``o*stride + t*dilation``; out-of-range reads are masked,
  src/ninetoothed/tensor.py:571-584)
* ``expand``  -- src/ninetoothed/tensor.py:288-321
* ``squeeze`` / ``unsqueeze`` -- src/ninetoothed/tensor.py:323-394
* ``permute`` -- src/ninetoothed/tensor.py:396-426
* ``flatten`` -- src/ninetoothed/tensor.py:428-484 (row-major merge)
* ``ravel``   -- src/ninetoothed/tensor.py:486-541 (levels merge into one)
* ``pad``     -- src/ninetoothed/tensor.py:543-569 (padding is masked)
* ``getitem`` -- src/ninetoothed/tensor.py:127-181, 677-729

``View.table`` has the layout of the reference's ``Tensor.eval()``
(src/ninetoothed/eval.py:15-58).  Pinned by the reference's own vectors in
``tests/golden/`` (tests/test_eval.py, tests/test_unsqueeze.py,
tests/test_getitem.py, tests/test_debugging.py of the reference).
"""

import math

import numpy as np


class View:
    def __init__(self, table, levels):
        self.table = np.asarray(table, dtype=np.intp)
        self.levels = list(levels)  # number of dims of each level, outermost first
        assert sum(self.levels) == self.table.ndim

    @staticmethod
    def of_shape(shape):
        """The identity view of a contiguous tensor."""
        size = int(np.prod(shape)) if len(shape) else 1
        return View(np.arange(size, dtype=np.intp).reshape(shape), [len(shape)])

    def _axis(self, level, dim=0):
        if level < 0:
            level += len(self.levels)
        ndim = self.levels[level]
        if dim < 0:
            dim += ndim
        return sum(self.levels[:level]) + dim

    def level_shape(self, level):
        start = self._axis(level)
        return self.table.shape[start : start + self.levels[level]]

    # ---- meta-operations (``level`` selects which level they act on) ----
    def tile(self, tile_shape, strides=None, dilation=None, floor_mode=False, level=0):
        ndim = self.levels[level]
        if strides is None:
            strides = [-1] * ndim
        if dilation is None:
            dilation = [1] * ndim
        table = self.table
        start = self._axis(level)
        inner_sizes = []
        for d in range(ndim):
            axis = start + d
            size = table.shape[axis]
            tile_size = size if tile_shape[d] == -1 else tile_shape[d]
            stride = tile_size if strides[d] == -1 else strides[d]
            spacing = dilation[d]
            span = size - spacing * (tile_size - 1) - 1
            count = span // stride + 1 if floor_mode else -(-span // stride) + 1
            count = max(count, 0)
            index = np.arange(count)[:, None] * stride + np.arange(tile_size)[None, :] * spacing
            valid = (index >= 0) & (index < size)
            padded = np.concatenate([table, np.full(table.shape[:axis] + (1,) + table.shape[axis + 1 :], -1, dtype=np.intp)], axis=axis)
            gathered = np.take(padded, np.where(valid, index, size).reshape(-1), axis=axis)
            # axis -> (count, tile_size); keep the outer part at `axis`, park the inner part at the end
            gathered = gathered.reshape(table.shape[:axis] + (count, tile_size) + table.shape[axis + 1 :])
            table = np.moveaxis(gathered, axis + 1, -1)
            inner_sizes.append(tile_size)
        # the parked inner axes (last ndim axes) become a new level right after `level`
        insert_at = start + ndim
        for d in range(ndim):
            table = np.moveaxis(table, table.ndim - ndim + d, insert_at + d)
        levels = self.levels[: level + 1] + [ndim] + self.levels[level + 1 :]
        return View(table, levels)

    def expand(self, shape, level=0):
        table = self.table
        start = self._axis(level)
        target = list(table.shape)
        for d, new_size in enumerate(shape):
            if new_size != -1:
                assert table.shape[start + d] == 1, "only singleton dimensions expand"
                target[start + d] = new_size
        return View(np.broadcast_to(table, target), self.levels)

    def squeeze(self, dims, level=0):
        dims = dims if isinstance(dims, tuple) else (dims,)
        axes = tuple(self._axis(level, d) for d in dims)
        for axis in axes:
            assert self.table.shape[axis] == 1
        levels = list(self.levels)
        levels[level] -= len(axes)
        return View(np.squeeze(self.table, axis=axes), levels)

    def unsqueeze(self, dim, level=0):
        ndim = self.levels[level]
        if dim < 0:
            dim += ndim + 1
        levels = list(self.levels)
        levels[level] += 1
        return View(np.expand_dims(self.table, self._axis(level) + dim), levels)

    def permute(self, dims, level=0):
        start = self._axis(level)
        order = list(range(self.table.ndim))
        for new, old in enumerate(dims):
            order[start + new] = start + old
        return View(np.transpose(self.table, order), self.levels)

    def flatten(self, start_dim=None, end_dim=None, level=0):
        ndim = self.levels[level]
        start_dim = 0 if start_dim is None else start_dim % ndim if start_dim < 0 else start_dim
        end_dim = ndim if end_dim is None else end_dim % ndim if end_dim < 0 else end_dim
        start = self._axis(level)
        shape = self.table.shape
        merged = math.prod(shape[start + start_dim : start + end_dim])
        new_shape = shape[: start + start_dim] + (merged,) + shape[start + end_dim :]
        levels = list(self.levels)
        levels[level] -= (end_dim - start_dim) - 1
        return View(np.ascontiguousarray(self.table).reshape(new_shape), levels)

    def ravel(self):
        return View(self.table, [self.table.ndim])

    def pad(self, pad, level=0):
        assert level == 0 and len(self.levels) == 1, "pad acts on an untiled tensor"
        return View(np.pad(self.table, pad, constant_values=-1), self.levels)

    def getitem(self, indices):
        assert len(self.levels) == 1
        table = self.table[indices]
        return View(table, [table.ndim])


def gather(flat_source, table, other):
    """Loads ``flat_source`` through an offset table; masked positions read ``other``."""
    safe = np.where(table >= 0, table, 0)
    values = flat_source[safe]
    if other is None:
        other = 0
    return np.where(table >= 0, values, np.asarray(other, dtype=values.dtype))


def scatter(flat_target, table, values):
    """Stores ``values`` through an offset table; masked positions are skipped."""
    mask = table >= 0
    flat_target[table[mask]] = values[mask]
