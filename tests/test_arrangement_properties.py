"""Random arrangements: the symbolic front-end, the brute-force oracle and the lowering agree.

A random chain of meta-operations is applied, step by step, to a symbolic ``Tensor`` and to an
``oracle.arrangement.View`` (offset tables, no algebra).  Two properties:

* ``Tensor.eval()`` equals the oracle's table (layout of the reference's ``Tensor.eval``,
  src/ninetoothed/eval.py:15-58);
* a clone program over that arrangement, lowered by ``ninetoothed_amd.mapping`` and executed by
  ``oracle.map_machine`` (same opcodes as the kernel), copies exactly the elements the table names.
"""

import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, assume, given, settings
from hypothesis import strategies as st

import ninetoothed_amd as ninetoothed
from ninetoothed_amd import Tensor, mapping
from ninetoothed_amd.make import _dtype_tag, _storage
from ninetoothed_amd.recognition import UnsupportedProgram
from oracle.arrangement import View
from oracle.map_machine import Machine


def _draw_chain(data, shape):
    """Returns a list of (name, args, kwargs) valid for a tensor of ``shape``; tracks the
    outermost level's shape with the oracle itself."""
    view = View.of_shape(shape)
    chain = []
    tiled = False
    for _ in range(data.draw(st.integers(1, 4), label="operations")):
        outer = view.level_shape(0)
        ndim = len(outer)
        choices = ["tile", "permute", "unsqueeze"]
        if not tiled:
            choices += ["pad", "getitem"]
        if ndim >= 2:
            choices.append("flatten")
        if any(size == 1 for size in outer):
            choices += ["expand", "squeeze"]
        if len(view.levels) >= 2:
            choices.append("ravel")
        if ndim == 0:
            choices = ["unsqueeze"]
        op = data.draw(st.sampled_from(choices), label="operation")
        args, kwargs = (), {}
        if op == "tile":
            if len(view.levels) >= 2 and data.draw(st.booleans()):
                break  # mostly one tile level: deeper nests are not what the executor runs
            tile_shape = tuple(data.draw(st.sampled_from((-1, 1, 2, 3, 4))) for _ in range(ndim))
            args = (tile_shape,)
            if data.draw(st.booleans()):
                kwargs["strides"] = tuple(data.draw(st.sampled_from((-1, 1, 2, 3))) for _ in range(ndim))
            if data.draw(st.booleans()):
                kwargs["dilation"] = tuple(data.draw(st.sampled_from((1, 2))) for _ in range(ndim))
            kwargs["floor_mode"] = data.draw(st.booleans())
            tiled = True
        elif op == "permute":
            args = (tuple(data.draw(st.permutations(range(ndim)))),)
        elif op == "unsqueeze":
            args = (data.draw(st.integers(0, ndim)),)
        elif op == "pad":
            args = (tuple((data.draw(st.integers(0, 2)), data.draw(st.integers(0, 2))) for _ in range(ndim)),)
        elif op == "getitem":
            indices = []
            for size in outer:
                start = data.draw(st.integers(0, max(size - 1, 0)))
                stop = data.draw(st.integers(start, size))
                step = data.draw(st.sampled_from((1, 2)))
                indices.append(slice(start, stop, step))
            args = (tuple(indices),)
        elif op == "flatten":
            start_dim = data.draw(st.integers(0, ndim - 2))
            end_dim = data.draw(st.integers(start_dim + 2, ndim))
            kwargs = {"start_dim": start_dim, "end_dim": end_dim}
        elif op == "expand":
            args = (tuple(data.draw(st.integers(2, 3)) if size == 1 and data.draw(st.booleans()) else -1 for size in outer),)
        elif op == "squeeze":
            args = (data.draw(st.sampled_from([d for d, size in enumerate(outer) if size == 1])),)
        view = _apply_view(view, op, args, kwargs)
        chain.append((op, args, kwargs))
        if view.table.size == 0 or view.table.size > 20000:
            break
    return chain


def _apply_view(view, op, args, kwargs):
    if op == "getitem":
        return view.getitem(*args)
    return getattr(view, op)(*args, **kwargs)


def _apply_tensor(tensor, op, args, kwargs):
    if op == "getitem":
        return tensor[args[0]]
    return getattr(tensor, op)(*args, **kwargs)


def _arranged(chain, shape, tensor=None):
    tensor = Tensor(shape=shape) if tensor is None else tensor
    view = View.of_shape(shape)
    for op, args, kwargs in chain:
        tensor = _apply_tensor(tensor, op, args, kwargs)
        view = _apply_view(view, op, args, kwargs)
    return tensor, view


_shapes = st.lists(st.integers(1, 7), min_size=1, max_size=3).map(tuple)


@settings(max_examples=400, deadline=None, suppress_health_check=[HealthCheck.too_slow, HealthCheck.data_too_large])
@given(shape=_shapes, data=st.data())
def test_eval_matches_the_offset_table_oracle(shape, data):
    chain = _draw_chain(data, shape)
    tensor, view = _arranged(chain, shape)
    assert np.array_equal(tensor.eval(), view.table), chain


def _clone_application(input, output):
    output = input  # noqa: F841


def _run_machine(kernel, args):
    env = kernel._environment(args, {}, check_device=False)
    flat = {p: arg.reshape(-1).numpy() for p, arg in enumerate(args)}
    for store in kernel.program.stores:
        built = mapping.build(store, kernel.types, args, env, lambda p: _dtype_tag(_storage(args, p).dtype), lambda p: 0)
        if built is not None:
            program, _, _, operand_params = built
            Machine(program, {slot: flat[p] for slot, p in enumerate(operand_params)}).run()


@settings(max_examples=400, deadline=None, suppress_health_check=[HealthCheck.too_slow, HealthCheck.data_too_large, HealthCheck.filter_too_much])
@given(shape=_shapes, data=st.data())
def test_lowered_clone_copies_what_the_table_names(shape, data):
    chain = _draw_chain(data, shape)
    _, view = _arranged(chain, shape)
    # (a tensor arranged down to zero dimensions is a call-time scalar to `make`, not an operand)
    assume(len(view.levels) <= 2 and view.table.size > 0 and len(view.level_shape(0)) > 0)

    def arrangement(input, output):
        return _arranged(chain, shape, input)[0], _arranged(chain, shape, output)[0]

    try:
        kernel = ninetoothed.make(arrangement, _clone_application, (Tensor(len(shape)), Tensor(len(shape))))
    except UnsupportedProgram:
        assume(False)
    source = torch.arange(1, int(np.prod(shape)) + 1, dtype=torch.float32).reshape(shape)
    out = torch.zeros(shape)
    try:
        _run_machine(kernel, (source, out))
    except UnsupportedProgram:
        assume(False)  # limits of the executor (variables, code length), not wrong results
    named = view.table[view.table >= 0]
    expected = np.zeros(int(np.prod(shape)), dtype=np.float32)
    expected[named] = named + 1
    assert np.array_equal(out.reshape(-1).numpy(), expected), chain


@pytest.mark.gpu
@settings(max_examples=60, deadline=None, derandomize=True, suppress_health_check=list(HealthCheck))
@given(shape=_shapes, data=st.data())
def test_clone_on_the_gpu_copies_what_the_table_names(shape, data):
    """The same property through ``launch_nt_map`` (specialised kernel and interpreter).  The numpy
    machine runs first: the device only sees index programs that stayed in bounds there."""
    import os

    chain = _draw_chain(data, shape)
    _, view = _arranged(chain, shape)
    assume(len(view.levels) <= 2 and view.table.size > 0 and len(view.level_shape(0)) > 0)

    def arrangement(input, output):
        return _arranged(chain, shape, input)[0], _arranged(chain, shape, output)[0]

    try:
        kernel = ninetoothed.make(arrangement, _clone_application, (Tensor(len(shape)), Tensor(len(shape))))
    except UnsupportedProgram:
        assume(False)
    source = torch.arange(1, int(np.prod(shape)) + 1, dtype=torch.float32).reshape(shape)
    named = view.table[view.table >= 0]
    expected = np.zeros(int(np.prod(shape)), dtype=np.float32)
    expected[named] = named + 1
    host_out = torch.zeros(shape)
    try:
        _run_machine(kernel, (source, host_out))
    except UnsupportedProgram:
        assume(False)
    assert np.array_equal(host_out.reshape(-1).numpy(), expected), chain
    for interpret in ("0", "1"):
        os.environ["NT_MAP_INTERPRET"] = interpret
        try:
            out = torch.zeros(shape, device="cuda")
            kernel(source.cuda(), out)
            assert np.array_equal(out.cpu().reshape(-1).numpy(), expected), (interpret, chain)
        finally:
            os.environ.pop("NT_MAP_INTERPRET", None)
