"""Symbolic tensors and the arrangement meta-operations.

A :class:`Tensor` describes how a program sees a source tensor: a stack of
levels (outermost level = the launch grid, innermost level = the tile a program
works on) and, for every level, how its indices lead back to indices of the
source.  The meta-operations ``tile``, ``expand``, ``squeeze``, ``unsqueeze``,
``permute``, ``flatten``, ``ravel``, ``pad`` and basic indexing follow the
reference's definitions (src/ninetoothed/tensor.py:199-569, 127-181, 677-729):
same arguments, same resulting shapes, same index arithmetic, and the same
masking rule -- a position is valid only if, at EVERY intermediate view it
passes through on the way to the source, its index lies inside that view
(src/ninetoothed/tensor.py:571-584).

Representation: every view is a node that points to the view(s) it was derived
from through :class:`_Link` records (plain data: a kind and its parameters).
Following the links from the levels of an arranged tensor up to the source and
summing the contributions that meet at a node gives the source index of an
element; collecting ``0 <= index < size`` at every node passed gives its mask.
"""

import itertools
import math

import numpy as np

from ninetoothed_amd.symbol import Symbol, evaluate


class _Link:
    """How the indices of a view contribute to the indices of ``parent``."""

    __slots__ = ("parent", "kind", "params")

    def __init__(self, parent, kind, params=None):
        self.parent = parent
        self.kind = kind
        self.params = params

    def apply(self, indices):
        kind, params = self.kind, self.params
        if kind == "scale":  # tile: outer index * stride, inner index * dilation
            return [index * factor for index, factor in zip(indices, params)]
        if kind == "expand":  # expanded dims do not move the parent index
            return [index if keep else Symbol(0) * index for index, keep in zip(indices, params)]
        if kind == "drop":  # unsqueeze: the new dim has no parent dim
            return [index for i, index in enumerate(indices) if i != params]
        if kind == "insert":  # squeeze: removed dims sit at index 0 in the parent
            iterator = iter(indices)
            return [Symbol(0) if i in params[1] else next(iterator) for i in range(params[0])]
        if kind == "permute":
            return [indices[params.index(dim)] for dim in range(len(params))]
        if kind == "unravel":  # flatten: decode one index into several
            start, sizes = params
            decoded = _unravel_index(indices[start], sizes)
            return list(indices[:start]) + decoded + list(indices[start + 1 :])
        if kind == "shift":  # pad: index - left padding
            return [index - amount for index, amount in zip(indices, params)]
        if kind == "slice":  # basic indexing: start + index * step
            dim, start, step = params
            result = list(indices)
            result[dim] = start + indices[dim] * step
            return result
        if kind == "segment":  # ravel: a run of the raveled dims belongs to one level
            start, stop = params
            return list(indices[start:stop])
        raise ValueError(f"Unknown link kind `{kind}`.")

    def substituted(self, parent, mapping):
        def sub(value):
            if isinstance(value, Symbol):
                return value.substitute(mapping)
            if isinstance(value, (list, tuple)):
                return type(value)(sub(item) for item in value)
            return value

        return _Link(parent, self.kind, sub(self.params))


def _unravel_index(index, sizes):
    """Row-major decode (reference: src/ninetoothed/tensor.py:773-790)."""
    strides = [1]
    for size in reversed(sizes[1:]):
        strides.append(size * strides[-1])
    strides.reverse()
    decoded = []
    for stride in strides:
        decoded.append(index // stride)
        index = index % stride
    return decoded


def _as_symbol(value):
    return value if isinstance(value, Symbol) else Symbol(value)


class Tensor:
    """A symbolic (possibly hierarchical) tensor.

    :param ndim: The number of dimensions.
    :param shape: The shape; ``None`` entries become size symbols.
    :param dtype: The element type, or the next inner level.
    :param jagged_dim: The dimension whose length differs per batch entry (a
        ``torch.jagged`` nested tensor is passed at call time; the batch is
        dimension 0).
    :param other: The value out-of-bounds positions read as.
    :param shape_options: Options for the size symbols (one dict, or one per dim).
    :param constexpr: Whether a zero-dimensional tensor is a call-time constant.
    :param value: The value of a constexpr tensor.
    :param name: The name of the tensor.
    """

    num_instances = 0
    _order = itertools.count()

    def __init__(
        self,
        ndim=None,
        shape=None,
        dtype=None,
        jagged_dim=None,
        other=None,
        shape_options=None,
        constexpr=None,
        value=None,
        name=None,
        source=None,
        target_dims=None,
        _links=None,
    ):
        self.dtype = dtype
        self.jagged_dim = jagged_dim

        if name is not None:
            self.name = name
        else:
            self.name = f"ninetoothed_tensor_{Tensor.num_instances}"

        if ndim is None and shape is None:
            raise ValueError("Either `ndim` or `shape` must be provided.")
        if ndim is None:
            ndim = len(shape)
        if shape is None:
            shape = (None,) * ndim
        if jagged_dim is not None and not 1 <= jagged_dim < ndim:
            raise ValueError("`jagged_dim` must name a dimension after the batch dimension.")

        if shape_options is None:
            shape_options = tuple({} for _ in range(ndim))
        if isinstance(shape_options, dict):
            shape_options = tuple(shape_options for _ in range(ndim))
        shape_options = tuple(options if options is not None else {} for options in shape_options)

        self.shape = tuple(
            size if size is not None else Symbol(self.size_string(i), **options)
            for i, (size, options) in enumerate(zip(shape, shape_options))
        )

        self.other = other

        if constexpr and self.ndim != 0:
            raise ValueError("`constexpr` can only be set for zero-dimensional tensors.")
        self.constexpr = constexpr
        if not constexpr and value is not None:
            raise ValueError("`value` can only be set for constexpr tensors.")
        self.value = value

        self.source = source if source is not None else self
        self.target_dims = tuple(target_dims) if target_dims is not None else tuple(range(self.ndim))

        self._links = list(_links) if _links is not None else []
        self._seq = next(Tensor._order)
        self._env = None  # substitutions attached by `subs`

        Tensor.num_instances += 1

    # ---- naming ----------------------------------------------------------
    def size_string(self, dim):
        return f"{self.name}_size_{dim}"

    def stride_string(self, dim):
        return f"{self.name}_stride_{dim}"

    def pointer_string(self):
        return f"{self.name}_pointer"

    # ---- basic properties --------------------------------------------------
    @property
    def shape(self):
        return self._shape

    @shape.setter
    def shape(self, value):
        self._shape = tuple(value)

    @property
    def ndim(self):
        return len(self._shape)

    def size(self, dim=None):
        return self.shape if dim is None else self.shape[dim]

    def innermost(self):
        current = self
        while isinstance(current.dtype, Tensor):
            current = current.dtype
        return current

    def levels(self):
        """The levels of this tensor, outermost first."""
        result = []
        current = self
        while isinstance(current, Tensor):
            result.append(current)
            current = current.dtype
        return result

    def _derive(self, shape, links, dtype="inherit", target_dims=None):
        return Tensor(
            shape=shape,
            dtype=self.dtype if isinstance(dtype, str) and dtype == "inherit" else dtype,
            source=self.source,
            target_dims=target_dims,
            _links=links,
        )

    # ---- meta-operations -----------------------------------------------------
    def tile(self, tile_shape, strides=None, dilation=None, floor_mode=False):
        """Tiles the tensor into a hierarchical tensor.

        :param tile_shape: The shape of a tile (``-1`` = the whole dim).
        :param strides: The interval at which tiles start (``-1`` = tile size).
        :param dilation: The spacing between the elements of a tile.
        :param floor_mode: Use floor instead of ceiling division for the
            number of tiles.
        :return: The outer level, whose ``dtype`` is the tile level.
        """

        if strides is None:
            strides = [-1] * len(tile_shape)
        if dilation is None:
            dilation = [1] * len(tile_shape)
        if not (len(tile_shape) == len(strides) == len(dilation) == self.ndim):
            raise ValueError("`tile_shape`, `strides` and `dilation` must have one entry per dimension.")

        outer_shape, outer_strides, inner_shape, inner_strides = [], [], [], []
        for size, tile_size, stride, spacing in zip(self.shape, tile_shape, strides, dilation):
            if tile_size == -1:
                tile_size = size
            if stride == -1:
                stride = tile_size
            span = size - spacing * (tile_size - 1) - 1
            if stride == 0:
                count = -1
            elif floor_mode:
                count = span // stride + 1
            else:
                count = (span + stride - 1) // stride + 1
            outer_shape.append(count)
            outer_strides.append(stride)
            inner_shape.append(tile_size)
            inner_strides.append(spacing)

        inner = self._derive(inner_shape, [_Link(self, "scale", tuple(inner_strides))])
        return self._derive(outer_shape, [_Link(self, "scale", tuple(outer_strides))], dtype=inner)

    def expand(self, shape):
        """Expands singleton dimensions (``-1`` keeps a dimension)."""
        keep = tuple(new_size == -1 for new_size in shape)
        new_shape = [size if new_size == -1 else new_size for size, new_size in zip(self.shape, shape)]
        return self._derive(new_shape, [_Link(self, "expand", keep)], target_dims=self.target_dims)

    def unsqueeze(self, dim):
        """Inserts a singleton dimension at ``dim``."""
        if dim < 0:
            dim += self.ndim + 1
        new_shape = list(self.shape)
        new_shape.insert(dim, 1)
        new_target_dims = list(self.target_dims)
        new_target_dims.insert(dim, None)
        return self._derive(new_shape, [_Link(self, "drop", dim)], target_dims=new_target_dims)

    def squeeze(self, dim):
        """Removes the given singleton dimension(s)."""
        dims = dim if isinstance(dim, tuple) else (dim,)
        dims = tuple(d + self.ndim if d < 0 else d for d in dims)
        new_shape = [size for i, size in enumerate(self.shape) if i not in dims]
        new_target_dims = [t for i, t in enumerate(self.target_dims) if i not in dims]
        return self._derive(new_shape, [_Link(self, "insert", (self.ndim, dims))], target_dims=new_target_dims)

    def permute(self, dims):
        """Permutes the dimensions: new dim ``i`` is old dim ``dims[i]``."""
        dims = tuple(dims)
        new_shape = [self.shape[dim] for dim in dims]
        return self._derive(new_shape, [_Link(self, "permute", dims)], target_dims=self.target_dims)

    def flatten(self, start_dim=None, end_dim=None):
        """Merges dims ``[start_dim, end_dim)`` of this level into one."""
        if start_dim is None:
            start_dim = 0
        if end_dim is None:
            end_dim = self.ndim
        if start_dim < 0:
            start_dim += self.ndim
        if end_dim < 0:
            end_dim += self.ndim
        merged = self.shape[start_dim:end_dim]
        new_shape = self.shape[:start_dim] + (math.prod(merged),) + self.shape[end_dim:]
        merged_targets = self.target_dims[start_dim:end_dim]
        new_target_dims = self.target_dims[:start_dim] + (merged_targets[-1] if merged_targets else None,) + self.target_dims[end_dim:]
        return self._derive(new_shape, [_Link(self, "unravel", (start_dim, tuple(merged)))], target_dims=new_target_dims)

    def ravel(self):
        """Flattens the hierarchy: all levels' dims become dims of one level."""
        new_shape, links, start = [], [], 0
        for level in self.levels():
            new_shape.extend(level.shape)
            links.append(_Link(level, "segment", (start, start + level.ndim)))
            start += level.ndim
        result = Tensor(shape=new_shape, other=self.source.other, source=self.source, _links=links)
        return result

    def pad(self, pad):
        """Pads every dimension with ``(before, after)`` positions."""
        new_shape = [size + (before + after) for size, (before, after) in zip(self.shape, pad)]
        return self._derive(new_shape, [_Link(self, "shift", tuple(before for before, _ in pad))], target_dims=self.target_dims)

    def _slice_dim(self, dim, start, stop=None, step=None):
        if dim < 0:
            dim += self.ndim
        if step is None:
            step = 1
        size = self.shape[dim]
        if start is None:
            start = 0 if step > 0 else size - 1
        if stop is None:
            stop = size if step > 0 else -1
        if isinstance(start, int) and start < 0:
            start += size
        if isinstance(stop, int) and (stop < 0 if step > 0 else stop < -1):
            stop += size
        new_shape = list(self.shape)
        new_shape[dim] = (stop - start + step - (1 if step > 0 else -1)) // step
        return self._derive(new_shape, [_Link(self, "slice", (dim, start, step))], target_dims=self.target_dims)

    def __getitem__(self, indices):
        """Basic indexing with ints, slices, ``None`` and one ``Ellipsis``."""
        if not isinstance(indices, tuple):
            indices = (indices,)
        if sum(index is Ellipsis for index in indices) > 1:
            raise ValueError("Only one `Ellipsis` is allowed.")
        num_effective = sum(index is not None and index is not Ellipsis for index in indices)
        if num_effective > self.ndim:
            raise IndexError(f"Index `{indices}` is out of bounds for tensor of shape `{self.shape}`.")

        expanded = []
        for index in indices:
            if index is Ellipsis:
                expanded.extend([slice(None)] * (self.ndim - num_effective))
            else:
                expanded.append(index)

        output, dim = self, 0
        for index in expanded:
            if index is None:
                output = output.unsqueeze(dim)
                dim += 1
            elif isinstance(index, int):
                output = output._slice_dim(dim, index, index + 1).squeeze(dim)
            elif isinstance(index, slice):
                output = output._slice_dim(dim, index.start, index.stop, index.step)
                dim += 1
            else:
                raise TypeError(f"Index `{index}` must be an `int`, `slice`, or `None`, not `{type(index).__name__}`.")
        return output

    # ---- index maps ----------------------------------------------------------
    def index_map(self):
        """Symbolic map from level indices to source indices.

        :return: ``(levels, index_symbols, source_indices, constraints)`` where
            ``index_symbols[l][d]`` is the index variable of dim ``d`` of level
            ``l``, ``source_indices[d]`` the resulting index into source dim
            ``d`` and ``constraints`` a list of ``(index, size)`` pairs, each
            standing for ``0 <= index < size``.
        """

        levels = self.levels()
        index_symbols = [[Symbol(f"ninetoothed_index_{l}_{d}") for d in range(level.ndim)] for l, level in enumerate(levels)]

        pending = {}
        for level, symbols in zip(levels, index_symbols):
            pending.setdefault(level._seq, (level, []))[1].append(list(symbols))

        constraints = []
        source_indices = None
        while pending:
            seq = max(pending)  # views are created after the views they derive from
            node, contributions = pending.pop(seq)
            indices = [_sum(parts) for parts in zip(*contributions)] if node.ndim else []
            for index, size in zip(indices, node.shape):
                constraints.append((_as_symbol(index), _as_symbol(size)))
            if not node._links:
                if node is not self.source:
                    raise ValueError("A level does not lead back to the source tensor.")
                source_indices = indices
                continue
            for link in node._links:
                pending.setdefault(link.parent._seq, (link.parent, []))[1].append(link.apply(indices))

        if source_indices is None:
            raise ValueError("The tensor does not lead back to its source.")
        return levels, index_symbols, source_indices, constraints

    def eval(self, subs=None):
        """Evaluates the tensor numerically.

        Returns an ``np.intp`` array with one axis per dim of every level
        (outermost level first) holding the flat offset, for a contiguous
        source, of the element each position refers to, or ``-1`` where the
        position is masked.  Same contract as the reference's ``Tensor.eval``
        (src/ninetoothed/eval.py:15-58).

        :param subs: Maps source :class:`Tensor` objects to ``{"shape": ...}``
            (or to a tensor with a concrete shape) and symbols to values.
        """

        if self.source.ndim == 0:
            return np.array(0, dtype=np.intp)

        env = dict(self._env or {})
        env.update(_environment(subs))
        if not any(name.startswith(self.source.name + "_size_") for name in env):
            env.update(_shape_environment(self.source, self.source.shape))

        levels, index_symbols, source_indices, constraints = self.index_map()
        # a tile larger than its tensor, stepped by less than its size, has a negative count: no tiles
        shape = [max(int(evaluate(size, env)), 0) for level in levels for size in level.shape]
        flat_symbols = [symbol for symbols in index_symbols for symbol in symbols]
        grids = np.ogrid[tuple(slice(0, extent) for extent in shape)] if shape else []
        for symbol, grid in zip(flat_symbols, grids):
            env[symbol.name] = grid

        source_shape = [int(evaluate(size, env)) for size in self.source.shape]
        strides = _contiguous_strides(source_shape)
        offsets = np.zeros(shape, dtype=np.intp)
        for index, stride in zip(source_indices, strides):
            offsets = offsets + np.asarray(evaluate(index, env), dtype=np.intp) * stride
        mask = np.ones(shape, dtype=bool)
        for index, size in constraints:
            value = np.asarray(evaluate(index, env))
            mask = mask & (value >= 0) & (value < evaluate(size, env))
        return np.where(mask, offsets, -1).astype(np.intp)

    def subs(self, subs):
        """Returns this tensor with the substitutions attached; its ``eval()``
        needs no further arguments (reference: src/ninetoothed/eval.py:61-100)."""

        env = dict(self._env or {})
        env.update(_environment(subs))
        mapping = {name: value for name, value in env.items() if not isinstance(value, np.ndarray)}

        clones = {}

        def clone(node):
            if node._seq in clones:
                return clones[node._seq]
            links = [link.substituted(clone(link.parent), mapping) for link in node._links]
            new_shape = [size.substitute(mapping) if isinstance(size, Symbol) else size for size in node.shape]
            new_shape = [size.value if isinstance(size, Symbol) and size.is_constant else size for size in new_shape]
            copy = Tensor.__new__(Tensor)
            copy.__dict__.update(node.__dict__)
            copy._shape = tuple(new_shape)
            copy._links = links
            clones[node._seq] = copy
            if not node._links:
                copy.source = copy
            return copy

        def rebuild(node):
            copy = clone(node)
            copy.source = clone(node.source)
            if isinstance(node.dtype, Tensor):
                copy.dtype = rebuild(node.dtype)
            copy._env = env
            return copy

        return rebuild(self)

    def __repr__(self):
        return f"Tensor(name={self.name!r}, shape={self.shape!r})"


def _sum(parts):
    total = parts[0]
    for part in parts[1:]:
        total = total + part
    return total


def _contiguous_strides(shape):
    strides = [1] * len(shape)
    for dim in range(len(shape) - 2, -1, -1):
        strides[dim] = strides[dim + 1] * shape[dim + 1]
    return strides


def _shape_environment(tensor, shape):
    env = {}
    shape = [int(size) if not isinstance(size, Symbol) else size for size in shape]
    for dim, size in enumerate(shape):
        if isinstance(size, Symbol):
            if not size.is_constant:
                raise ValueError(f"The size of dimension {dim} of `{tensor.name}` is not known; pass it in `subs`.")
            size = size.value
        env[tensor.size_string(dim)] = size
    for dim, stride in enumerate(_contiguous_strides([env[tensor.size_string(d)] for d in range(len(shape))])):
        env[tensor.stride_string(dim)] = stride
    return env


def _environment(subs):
    env = {}
    if not subs:
        return env
    for key, value in subs.items():
        if isinstance(key, Tensor):
            shape = value.shape if isinstance(value, Tensor) else value["shape"]
            env.update(_shape_environment(key.source, shape))
        elif isinstance(key, Symbol):
            env[key.name] = value
        else:
            raise TypeError(f"Cannot substitute `{key!r}`.")
    return env
