"""Recognises which of the supported programs an (arrangement, application)
pair is, and extracts what the gfx950 kernels need to run it.

Two independent checks have to agree:

* the application's dataflow graph must equal the graph of one of the programs
  in :mod:`ninetoothed_amd.programs` (digest comparison, see
  :mod:`ninetoothed_amd.tracing`);
* the arrangement's index maps, evaluated for the sizes and strides of the
  call, must have the structure that program's kernel implements (strided
  matrices, the im2col view of conv2d, row segments, [batch, head, seq, dim]
  tiles), including its masks.

What the reference does at this point is generate Triton code for arbitrary
programs (src/ninetoothed/generation.py:46-133); here anything that is not
recognised is reported, not approximated.
"""

import functools

from ninetoothed_amd import programs
from ninetoothed_amd.affine import Affine, NotAffine, Ranges
from ninetoothed_amd.symbol import Symbol, evaluate
from ninetoothed_amd.symbolic_int import constant_difference, integer, is_symbolic, same_structure
from ninetoothed_amd.tensor import Tensor
from ninetoothed_amd.tracing import Carried, Dim, LoopVar, Node, Program, TensorRef, TracingError, trace


class UnsupportedProgram(NotImplementedError):
    """The program is not one this build has a kernel for."""


# ---- application dictionary ---------------------------------------------------


def _trace_template(cls, application, arrangement=None, tensors=None):
    types = (arrangement or cls.arrangement)(*(tensors if tensors is not None else cls.tensors()))
    types = types if isinstance(types, tuple) else (types,)
    return trace(application, types).digest


@functools.lru_cache(maxsize=None)
def known_applications():
    """Maps application digests to ``(kind, details)``."""
    table = {}
    m, a, s, t = programs.matmul, programs.addmm, programs.softmax, programs.attention
    table[_trace_template(m, m.application)] = ("matmul", {"cast": None})
    table[_trace_template(m, m.application_with_cast)] = ("matmul", {"cast": "fp16"})
    table[_trace_template(m, m.application_with_bfloat16_cast)] = ("matmul", {"cast": "bf16"})
    table[_trace_template(a, a.application)] = ("addmm", {"cast": "fp16"})
    table[_trace_template(a, a.application_bfloat16)] = ("addmm", {"cast": "bf16"})
    table[_trace_template(s, s.application)] = ("softmax", {})
    table[_trace_template(t, t.application)] = ("attention", {"scale": False})
    table[_trace_template(t, t.application_with_scale, t.arrangement_with_scale, t.tensors(True))] = ("attention", {"scale": True})
    return table


def identify(application, types):
    """Returns ``(kind, details, program)`` for a traced application."""
    try:
        program = trace(application, types)
    except TracingError as error:
        raise UnsupportedProgram(f"The application could not be traced: {error}") from error
    entry = known_applications().get(program.digest)
    if entry is None:
        from ninetoothed_amd import mapping  # imports this module

        try:
            mapping.check_application(program)
        except UnsupportedProgram as error:
            fused = match_gemm_with_epilogue(program, types)
            if fused is not None:
                return "gemm_epilogue", fused, program
            raise UnsupportedProgram(
                "The application is not one of the programs this build has kernels for "
                "(matmul, addmm, row softmax, attention forward, conv2d as matmul) and not an element-wise / reducing "
                f"tile map either ({error}).  Its dataflow graph:\n" + program.describe()
            ) from error
        return "map", {}, program
    return entry[0], entry[1], program


# ---- a matrix product followed by element-wise work on the accumulator ---------------------------


def _is_accumulation(node):
    """``loop_out`` of `acc = zeros(...); for k in range(lhs.shape[0]): acc += dot(lhs[k], rhs[k])`:
    returns the parameter positions (lhs, rhs), or None."""
    if not (isinstance(node, Node) and node.op == "loop_out" and node.args[1] == 0):
        return None
    loop = node.args[0]
    if not (isinstance(loop, Node) and loop.op == "loop" and len(loop.args[1]) == 1 and len(loop.args[2]) == 1):
        return None
    init, body = loop.args[1][0], loop.args[2][0]
    if not (isinstance(init, Node) and init.op == "zeros"):
        return None
    if not (isinstance(body, Node) and body.op == "add" and len(body.args) == 2):
        return None
    carried = [arg for arg in body.args if isinstance(arg, Carried)]
    products = [arg for arg in body.args if isinstance(arg, Node) and arg.op == "dot" and len(arg.args) == 2]
    if len(carried) != 1 or len(products) != 1:
        return None
    operands = []
    for factor in products[0].args:
        if not (isinstance(factor, Node) and factor.op == "load" and isinstance(factor.args[0], TensorRef)):
            return None
        ref = factor.args[0]
        if ref.level != 2 or len(ref.indices) != 1 or not isinstance(ref.indices[0], LoopVar):
            return None
        operands.append(ref.param)
    extent = loop.args[0]
    if not (isinstance(extent, Dim) and extent.param == operands[0] and extent.level == 1 and extent.dim == 0):
        return None
    return tuple(operands)


def match_gemm_with_epilogue(program, types):
    """A single store whose value is element-wise work on one matmul accumulator (bias, activation,
    scaling, a residual ...).  Returns ``{"lhs", "rhs", "output", "accumulator"}`` (parameter
    positions and the accumulator node) when, with the accumulator replaced by a tile of a new
    tensor arranged like the output, the rest is a tile map; else None."""
    from ninetoothed_amd import mapping

    if len(program.stores) != 1 or not isinstance(program.stores[0][0], TensorRef):
        return None
    ref, value = program.stores[0]
    found = {}

    def visit(item):
        if isinstance(item, Node):
            operands = _is_accumulation(item)
            if operands is not None:
                found[item.digest] = (item, operands)
                return
            for arg in item.args:
                visit(arg)
        elif isinstance(item, (tuple, list)):
            for arg in item:
                visit(arg)

    visit(value)
    if len(found) != 1:
        return None
    (accumulator, (lhs, rhs)), = found.values()
    if ref.level != 1 or not ref.is_tile or ref.param in (lhs, rhs):
        return None
    stand_in = TensorRef(len(types), ref.tensor, 1)
    epilogue = substitute(value, accumulator.digest, Node("load", stand_in))
    candidate = Program(program.params + [("tensor", False)], [(ref, epilogue)])
    try:
        mapping.check_application(candidate)
    except UnsupportedProgram:
        return None
    return {"lhs": lhs, "rhs": rhs, "output": ref.param, "epilogue": candidate}


def substitute(value, digest, replacement):
    """``value`` with every node of that digest replaced."""
    if isinstance(value, Node):
        if value.digest == digest:
            return replacement
        return Node(value.op, *[substitute(arg, digest, replacement) for arg in value.args])
    if isinstance(value, tuple):
        return tuple(substitute(item, digest, replacement) for item in value)
    if isinstance(value, list):
        return [substitute(item, digest, replacement) for item in value]
    return value


# ---- arrangement analysis -------------------------------------------------------


class Operand:
    """The index map of one arranged tensor for one call."""

    def __init__(self, tensor, env):
        self.tensor = tensor
        self.env = env
        levels, symbols, source_indices, constraints = tensor.index_map()
        self.levels = levels
        self.names = [[symbol.name for symbol in level_symbols] for level_symbols in symbols]
        extents = {}
        for level, level_names in zip(levels, self.names):
            for name, size in zip(level_names, level.shape):
                extents[name] = integer(evaluate(size, env))
        self.extents = extents
        self.empty = any(extent <= 0 for extent in extents.values())
        self.ranges = Ranges({name: max(extent, 1) for name, extent in extents.items()})
        source = tensor.source
        self.source_shape = [integer(evaluate(size, env)) for size in source.shape]
        self.source_strides = [integer(env[source.stride_string(d)]) for d in range(source.ndim)]
        try:
            self.indices = [self.ranges.convert(index, env) for index in source_indices]
            self.constraints = [(self.ranges.convert(index, env), integer(evaluate(size, env))) for index, size in constraints]
        except NotAffine as error:
            raise UnsupportedProgram(f"Index map of `{source.name}` is not div/mod-affine: {error}") from error
        self._prune()

    def _prune(self):
        """Drops the constraints the variable ranges already guarantee."""
        remaining = []
        for index, size in self.constraints:
            lo, hi = self.ranges.interval(index)
            # sizes only known at launch: the check stays unless the bounds show for every call that it holds
            if is_symbolic(lo, hi, size):
                below, above = constant_difference(lo, 0), constant_difference(hi, size)
                if below is not None and below >= 0 and above is not None and above < 0:
                    continue
                if not any(same_structure((index.key(), size), (known.key(), bound)) for known, bound in remaining):
                    remaining.append((index, size))
            elif (lo < 0 or hi >= size) and (index, size) not in remaining:
                remaining.append((index, size))
        self.constraints = remaining

    def fuse(self, outer, inner, fused):
        block = self.extents[inner]
        exprs = self.indices + [index for index, _ in self.constraints]
        try:
            exprs = self.ranges.fuse(exprs, outer, inner, block, fused)
        except NotAffine as error:
            raise UnsupportedProgram(f"Arrangement of `{self.tensor.source.name}`: {error}") from error
        n = len(self.indices)
        self.indices = exprs[:n]
        self.constraints = [(expr, size) for expr, (_, size) in zip(exprs[n:], self.constraints)]
        return block

    def settle(self):
        """Uses constraints of the form ``variable < bound`` to tighten the
        variable's range, re-normalises, and drops constraints that the
        ranges already guarantee.  Returns the remaining constraints."""

        changed = True
        while changed:
            changed = False
            for index, size in self.constraints:
                if index.const == 0 and len(index.terms) == 1:
                    (atom, coef), = index.terms.items()
                    if atom[0] == "var" and coef == 1:
                        lo, hi = self.ranges.bounds[atom[1]]
                        if hi > size - 1:
                            self.ranges.bounds[atom[1]] = (lo, max(size - 1, lo))
                            changed = True
            if changed:
                self.indices = [self.ranges.rewrite(index, {}) for index in self.indices]
                self.constraints = [(self.ranges.rewrite(index, {}), size) for index, size in self.constraints]
        self._prune()
        return self.constraints

    def extent(self, name):
        lo, hi = self.ranges.bounds[name]
        return hi - lo + 1

    def rename(self, old, new):
        """Gives a variable the name the operands of a program share (``b`` for a batch index)."""
        self.ranges.bounds[new] = self.ranges.bounds.get(old, (0, 0))
        self.extents[new] = self.extents.get(old, 1)
        substitution = {old: Affine.var(new)}
        self.indices = [self.ranges.rewrite(index, substitution) for index in self.indices]
        self.constraints = [(self.ranges.rewrite(index, substitution), size) for index, size in self.constraints]

    def offset(self):
        total = Affine(0)
        for index, stride in zip(self.indices, self.source_strides):
            total = total + index * stride
        return total

    def require_absent(self, name):
        if self.extents.get(name, 1) <= 1:
            return
        for expr in self.indices + [index for index, _ in self.constraints]:
            if name in expr.variables():
                raise UnsupportedProgram(f"`{self.tensor.source.name}` depends on a grid dimension it should be expanded along.")


def _level_shape(operand, expected):
    actual = [len(names) for names in operand.names]
    if actual != expected:
        raise UnsupportedProgram(
            f"`{operand.tensor.source.name}` is arranged into levels with {actual} dimensions; this program needs {expected}."
        )


class Strided2d:
    """offset(row, col) = base + row * row_stride + col * col_stride."""

    def __init__(self, rows, cols, base, row_stride, col_stride):
        self.rows, self.cols, self.base = rows, cols, base
        self.row_stride, self.col_stride = row_stride, col_stride


def _strided(operand, row, col):
    if operand.constraints:
        return None
    offset = operand.offset()
    if not offset.is_linear() or (offset.variables() - {row, col}):
        return None
    return Strided2d(operand.extent(row), operand.extent(col), offset.const, offset.coef(row), offset.coef(col))


class Strided3d(Strided2d):
    """offset(batch, row, col) = base + batch * batch_stride + row * row_stride + col * col_stride."""

    def __init__(self, batches, rows, cols, base, batch_stride, row_stride, col_stride):
        super().__init__(rows, cols, base, row_stride, col_stride)
        self.batches, self.batch_stride = batches, batch_stride


def _strided_batched(operand, row, col):
    if operand.constraints:
        return None
    offset = operand.offset()
    if not offset.is_linear() or (offset.variables() - {"b", row, col}):
        return None
    return Strided3d(operand.extent("b"), operand.extent(row), operand.extent(col), offset.const, offset.coef("b"), offset.coef(row), offset.coef(col))


def _analyze_batched_gemm(lhs, rhs, out):
    """The matmul application under an arrangement with a leading batch dimension tiled by 1: grid
    (batch, blocks of M, blocks of N), the operands' K blocks on a middle level (the batched product of
    the reference's users; src/ninetoothed/generation.py:46-133 generates a kernel for any such
    arrangement).  Returns ``("batched", {...})``."""
    _level_shape(lhs, [3, 1, 2])
    _level_shape(rhs, [3, 1, 2])
    _level_shape(out, [3, 2])
    operands = [lhs, rhs, out]
    if any(operand.empty for operand in operands):
        return "empty", {}
    blocks = {}
    blocks["m"] = lhs.fuse(lhs.names[0][1], lhs.names[2][0], "m")
    blocks["k"] = lhs.fuse(lhs.names[1][0], lhs.names[2][1], "k")
    rhs_block_k = rhs.fuse(rhs.names[1][0], rhs.names[2][0], "k")
    blocks["n"] = rhs.fuse(rhs.names[0][2], rhs.names[2][1], "n")
    if out.fuse(out.names[0][1], out.names[1][0], "m") != blocks["m"] or out.fuse(out.names[0][2], out.names[1][1], "n") != blocks["n"]:
        raise UnsupportedProgram("Operands are tiled with different block sizes.")
    if rhs_block_k != blocks["k"]:
        raise UnsupportedProgram("`lhs` and `rhs` are tiled with different block sizes along K.")
    for operand in operands:
        operand.rename(operand.names[0][0], "b")
        operand.settle()
    lhs.require_absent(lhs.names[0][2])
    rhs.require_absent(rhs.names[0][1])
    if lhs.extents[lhs.names[1][0]] != rhs.extents[rhs.names[1][0]]:
        raise UnsupportedProgram("`lhs` and `rhs` disagree on the number of K blocks.")
    a, b, c = _strided_batched(lhs, "m", "k"), _strided_batched(rhs, "k", "n"), _strided_batched(out, "m", "n")
    if not (a and b and c):
        raise UnsupportedProgram("The operands of the batched product are not plain strided matrices per batch entry.")
    if a.cols != b.rows:
        raise UnsupportedProgram(f"Inner dimensions differ: {a.cols} and {b.rows}.")
    batch, m, n, k = c.batches, c.rows, c.cols, a.cols
    if a.rows < m or b.cols < n or a.batches != batch or b.batches != batch:
        raise UnsupportedProgram("The output is larger than the product of the operands.")
    return "batched", {"batch": batch, "m": m, "n": n, "k": k, "a": a, "b": b, "c": c, "blocks": blocks}


def analyze_gemm(lhs_type, rhs_type, out_type, env, input_type=None):
    """Returns ``("strided", {...})``, ``("batched", {...})`` or ``("conv2d", {...})``."""
    lhs, rhs, out = Operand(lhs_type, env), Operand(rhs_type, env), Operand(out_type, env)
    if input_type is None and len(out.names[0]) == 3:
        return _analyze_batched_gemm(lhs, rhs, out)
    operands = [lhs, rhs, out]
    _level_shape(lhs, [2, 1, 2])
    _level_shape(rhs, [2, 1, 2])
    _level_shape(out, [2, 2])
    inp = None
    if input_type is not None:
        inp = Operand(input_type, env)
        _level_shape(inp, [2, 2])
        operands.append(inp)
    if any(operand.empty for operand in operands):
        return "empty", {}

    blocks = {}
    blocks["m"] = lhs.fuse(lhs.names[0][0], lhs.names[2][0], "m")
    blocks["k"] = lhs.fuse(lhs.names[1][0], lhs.names[2][1], "k")
    rhs_block_k = rhs.fuse(rhs.names[1][0], rhs.names[2][0], "k")
    blocks["n"] = rhs.fuse(rhs.names[0][1], rhs.names[2][1], "n")
    for operand in (out, inp):
        if operand is not None:
            block_m = operand.fuse(operand.names[0][0], operand.names[1][0], "m")
            block_n = operand.fuse(operand.names[0][1], operand.names[1][1], "n")
            if block_m != blocks["m"] or block_n != blocks["n"]:
                raise UnsupportedProgram("Operands are tiled with different block sizes.")
    if rhs_block_k != blocks["k"]:
        raise UnsupportedProgram("`lhs` and `rhs` are tiled with different block sizes along K.")
    for operand in operands:
        operand.settle()
    lhs.require_absent(lhs.names[0][1])
    rhs.require_absent(rhs.names[0][0])

    if lhs.extents[lhs.names[1][0]] != rhs.extents[rhs.names[1][0]]:
        raise UnsupportedProgram("`lhs` and `rhs` disagree on the number of K blocks.")

    a, b, c = _strided(lhs, "m", "k"), _strided(rhs, "k", "n"), _strided(out, "m", "n")
    i = _strided(inp, "m", "n") if inp is not None else None
    if a and b and c and (inp is None or i):
        if a.cols != b.rows:
            raise UnsupportedProgram(f"Inner dimensions differ: {a.cols} and {b.rows}.")
        # rows / columns beyond the output are never stored; beyond A / B they read as zero
        m, n, k = c.rows, c.cols, a.cols
        if a.rows < m or b.cols < n or (i is not None and (i.rows < m or i.cols < n)):
            raise UnsupportedProgram("The output is larger than the product of the operands.")
        return "strided", {"m": m, "n": n, "k": k, "a": a, "b": b, "c": c, "input": i, "blocks": blocks}

    if inp is None:
        conv = _match_conv2d(lhs, rhs, out)
        if conv is not None:
            conv["blocks"] = blocks
            return "conv2d", conv
    raise UnsupportedProgram("The operands are neither plain strided matrices nor the conv2d views this build supports.")


def _match_conv2d(lhs, rhs, out):
    """Checks that lhs / rhs / out are the implicit-GEMM views of x[N,C,H,W], w[K,C,R,S], y[N,K,P,Q]: GEMM row
    (image, out_y, out_x) and k (channel, f_y, f_x) read x[image, channel, out_y * stride_h + f_y * dilation_h -
    pad_h, out_x * stride_w + f_x * dilation_w - pad_w], zero outside (`tile` with strides and dilation over the
    padded input, src/ninetoothed/tensor.py:199-286)."""

    if len(lhs.indices) != 4 or len(rhs.indices) != 4 or len(out.indices) != 4:
        return None
    N, C, H, W = lhs.source_shape
    K, C2, R, S = rhs.source_shape
    N2, K2, P, Q = out.source_shape
    if C != C2 or N != N2 or K != K2 or min(P, Q, R, S) <= 0:
        return None
    pad_h, pad_w = -lhs.indices[2].const, -lhs.indices[3].const
    if pad_h < 0 or pad_w < 0:
        return None
    if lhs.extent("m") != N * P * Q or lhs.extent("k") != C * R * S:
        return None
    if out.extent("m") != N * P * Q or out.extent("n") != K or rhs.extent("k") != C * R * S or rhs.extent("n") != K:
        return None
    if lhs.tensor.source.other not in (None, 0, 0.0):
        return None  # padding must read as zero

    def row_parts(ranges):  # GEMM row -> (image, out_y, out_x)
        m = Affine.var("m") if "m" in ranges.bounds and ranges.bounds["m"][1] > 0 else Affine(0)
        return ranges.floordiv(m, P * Q), ranges.floordiv(ranges.mod(m, P * Q), Q), ranges.mod(m, Q)

    def k_parts(ranges):  # GEMM k -> (channel, filter_y, filter_x)
        k = Affine.var("k") if ranges.bounds["k"][1] > 0 else Affine(0)
        return ranges.floordiv(k, R * S), ranges.floordiv(ranges.mod(k, R * S), S), ranges.mod(k, S)

    def column(ranges):
        return Affine.var("n") if ranges.bounds["n"][1] > 0 else Affine(0)

    def step(index, part):
        """The factor `part` (an output coordinate or a tap coordinate) carries in a source index: the window's
        stride or the dilation.  1 when the part is constant (a single position), None when it is not plain."""
        if part.is_const():
            return 1
        if part.const != 0 or len(part.terms) != 1:
            return None
        (atom, unit), = part.terms.items()
        factor = index.terms.get(atom, 0)
        return factor // unit if unit and factor % unit == 0 and factor // unit >= 1 else None

    image, out_y, out_x = row_parts(lhs.ranges)
    channel, f_y, f_x = k_parts(lhs.ranges)
    stride_h, dil_h = step(lhs.indices[2], out_y), step(lhs.indices[2], f_y)
    stride_w, dil_w = step(lhs.indices[3], out_x), step(lhs.indices[3], f_x)
    if None in (stride_h, dil_h, stride_w, dil_w):
        return None
    expected_x = [image, channel, out_y * stride_h + f_y * dil_h - pad_h, out_x * stride_w + f_x * dil_w - pad_w]
    channel, f_y, f_x = k_parts(rhs.ranges)
    expected_w = [column(rhs.ranges), channel, f_y, f_x]
    image, out_y, out_x = row_parts(out.ranges)
    expected_y = [image, column(out.ranges), out_y, out_x]
    if lhs.indices != expected_x or rhs.indices != expected_w or out.indices != expected_y:
        return None
    # windows: as many as fit, or one more that hangs over the edge (`tile` rounds up unless `floor_mode`)
    fits = True
    for size, pad, taps, dil, stride, count in ((H, pad_h, R, dil_h, stride_h, P), (W, pad_w, S, dil_w, stride_w, Q)):
        span = size + 2 * pad - dil * (taps - 1) - 1
        if span < 0 or count not in (span // stride + 1, -(-span // stride) + 1):
            return None
        fits = fits and count == span // stride + 1
    # the masks of the source (and, implied by them, of the padded view a hanging window runs out of)
    allowed = [(expected_x[2], H), (expected_x[3], W), (expected_x[2] + pad_h, H + 2 * pad_h), (expected_x[3] + pad_w, W + 2 * pad_w)]
    if any(constraint not in allowed for constraint in lhs.constraints) or rhs.constraints or out.constraints:
        return None
    required = [(expected_x[2], H), (expected_x[3], W)]
    for constraint in required:
        lo, hi = lhs.ranges.interval(constraint[0])
        if (lo < 0 or hi >= constraint[1]) and constraint not in lhs.constraints:
            return None  # positions outside the input must be masked (they read as zero)
    return {"fits": fits, "pad_h": pad_h, "pad_w": pad_w, "stride_h": stride_h, "stride_w": stride_w, "dilation_h": dil_h, "dilation_w": dil_w,
            "m": N * P * Q, "n": K, "k": C * R * S}


def analyze_softmax(input_type, output_type, env):
    result = {}
    for role, tensor in (("input", input_type), ("output", output_type)):
        operand = Operand(tensor, env)
        _level_shape(operand, [2, 2])
        if operand.empty:
            return "empty", {}
        (g0, g1), (t0, t1) = operand.names
        if operand.extents[t0] != 1:
            raise UnsupportedProgram("Softmax tiles must be one row high.")
        block = operand.extents[t1]
        rows, cols = operand.source_shape
        row_index = Affine.var(g0) if operand.extents[g0] > 1 else Affine(0)
        col_index = (Affine.var(g1) * block if operand.extents[g1] > 1 else Affine(0)) + (Affine.var(t1) if block > 1 else Affine(0))
        if operand.indices != [row_index, col_index] or operand.extents[g0] != rows:
            raise UnsupportedProgram(f"`{tensor.source.name}` is not tiled into row segments.")
        remaining = operand.settle()
        if any(constraint != (col_index, cols) for constraint in remaining):
            raise UnsupportedProgram(f"`{tensor.source.name}` carries a mask this kernel does not implement.")
        if role == "input" and remaining and tensor.source.other != float("-inf"):
            raise UnsupportedProgram("Row segments are padded, but out-of-bounds input does not read as -inf.")
        if operand.extents[g1] * block < cols:
            raise UnsupportedProgram("The tiles do not cover the rows.")
        result[role] = {"rows": rows, "cols": cols, "block": block, "row_stride": operand.source_strides[0], "col_stride": operand.source_strides[1]}
    if (result["input"]["rows"], result["input"]["cols"], result["input"]["block"]) != (
        result["output"]["rows"],
        result["output"]["cols"],
        result["output"]["block"],
    ):
        raise UnsupportedProgram("Input and output of the softmax are tiled differently.")
    return "softmax", result


def analyze_attention(q_type, k_type, v_type, o_type, env):
    info = {}
    q_blocks = None
    for role, tensor in (("q", q_type), ("k", k_type), ("v", v_type), ("o", o_type)):
        operand = Operand(tensor, env)
        if operand.empty:
            return "empty", {}
        if len(operand.source_shape) != 4:
            raise UnsupportedProgram("Attention operands must be [batch, heads, seq, head_dim].")
        if role in ("q", "o"):
            _level_shape(operand, [4, 2])
            grid, tile = operand.names
            operand.fuse(grid[2], tile[0], "s")
            seq_blocks = operand.extents[grid[2]]
        else:
            _level_shape(operand, [4, 1, 2])
            grid, (loop,), tile = operand.names
            operand.fuse(loop, tile[0], "s")
            seq_blocks = operand.extents[grid[2]]
        operand.settle()
        if role in ("k", "v"):
            operand.require_absent(grid[2])
        batch, heads, seq, dim = operand.source_shape
        if operand.extents[tile[1]] != dim or operand.extents[grid[3]] != 1:
            raise UnsupportedProgram("Attention tiles must span the whole head dimension.")
        expected = [
            Affine.var(grid[0]) if batch > 1 else Affine(0),
            Affine.var(grid[1]) if heads > 1 else Affine(0),
            Affine.var("s") if operand.extent("s") > 1 else Affine(0),
            Affine.var(tile[1]) if dim > 1 else Affine(0),
        ]
        if operand.indices != expected or operand.constraints:
            raise UnsupportedProgram(f"`{tensor.source.name}` is not tiled along the sequence dimension only.")
        if operand.extents[grid[0]] != batch or operand.extents[grid[1]] != heads or operand.extent("s") != seq:
            raise UnsupportedProgram(f"The grid of `{tensor.source.name}` does not cover batch, heads and sequence.")
        if q_blocks is None:
            q_blocks = seq_blocks
        elif seq_blocks != q_blocks:
            raise UnsupportedProgram("K / V are not expanded to the number of query blocks.")
        if role in ("k", "v") and tensor.source.other not in (None, 0, 0.0):
            raise UnsupportedProgram("Out-of-bounds K / V must read as zero.")
        info[role] = {"shape": operand.source_shape, "strides": operand.source_strides}
    return "attention", info


def unbound_meta_symbols(types):
    """Meta (tunable) symbols that appear in the arranged tensors."""
    found = {}

    def scan(value):
        if isinstance(value, Symbol):
            for symbol in value.names():
                if symbol.meta:
                    found[symbol.name] = symbol
        elif isinstance(value, (tuple, list)):
            for item in value:
                scan(item)

    seen = set()

    def visit(node):
        if node._seq in seen:
            return
        seen.add(node._seq)
        scan(node.shape)
        for link in node._links:
            scan(link.params)
            visit(link.parent)
        if isinstance(node.dtype, Tensor):
            visit(node.dtype)

    for tensor in types:
        if isinstance(tensor, Tensor):
            visit(tensor)
    return found
