"""Lowers element-wise / reducing tile programs to the interpreter kernel of
``libnt_hip.so`` (``launch_nt_map``).

The reference generates a Triton kernel for any arrange-and-apply pair
(src/ninetoothed/generation.py:28-837).  Programs that are none of the
recognised ones (matmul, addmm, softmax, attention, conv2d) run here if their
application is a *tile map*: every store assigns, to a tile of an output
parameter, an expression over whole tiles of the other parameters, call-time
scalars and constants, with at most one ``ntl.max`` / ``ntl.min`` / ``ntl.sum``
reduction (the programs of the reference's tests/test_add.py, test_clone.py,
test_pad.py, test_pow.py, test_dropout.py, test_max_pool2d.py,
test_generation.py:139-151).  Besides tiles, a value may be read from, and a
store may go to, elements of a whole tensor picked by computed indices
(``x.source[rows, columns]``, masked to the tensor's bounds as
src/ninetoothed/tensor.py:571-584 does) or by a raw pointer
(``ntl.load / ntl.store / ntl.atomic_add`` on ``x.source.data_ptr() + offsets``,
unmasked) -- tests/test_clone.py:23-37 and tests/test_data_ptr.py:17-18.

Two lowerings happen per call signature:

* every operand's index map (:meth:`Tensor.index_map`, normal form of
  :mod:`ninetoothed_amd.affine`) becomes a stack program over shared index
  variables -- the launch grid's dimensions, the output tile's dimensions, the
  reduced dimensions -- with the arrangement's masks as range checks;
* the dataflow graph of the stored value becomes a stack program over
  doubles, with a rounding step wherever the reference holds the value in a
  narrower type (type promotion as Triton applies it to the generated code: a
  Python literal takes the tile's type, a run-time ``float`` argument is fp32,
  mixed half types promote to fp32, ``/`` on integers gives fp32, sums of
  fp16 / bf16 tiles accumulate in fp32).
"""

import ctypes

from ninetoothed_amd import runtime
from ninetoothed_amd.affine import Affine
from ninetoothed_amd.recognition import Operand, UnsupportedProgram
from ninetoothed_amd.symbol import evaluate
from ninetoothed_amd.symbolic_int import integer, is_symbolic, plain, same
from ninetoothed_amd.tracing import Dim, ElementType, Node, ScalarParam, SourceDim, SourceStride, TensorRef

MAX_OPERANDS = 8
MAX_VARS = 16
MAX_INDEX_CODE = 320
MAX_INDEX_CONSTANTS = 96
MAX_SEGMENTS = 16
MAX_VALUE_CODE = 128
MAX_VALUE_CONSTANTS = 32
MAX_PHASES = 4

I_END, I_CONST, I_VAR, I_MULC, I_ADD, I_DIVC, I_MODC, I_CHECK = range(8)

_VALUE_OPS = (
    "LOAD CONST OFFSET ADD SUB MUL DIV FLOORDIV MOD POW MAX MIN LT LE GT GE EQ NE AND OR "
    "NEG NOT ABS EXP EXP2 LOG LOG2 SQRT RSQRT SIGMOID TANH SIN COS FLOOR CEIL WHERE ROUND RAND SETVAR REDUCED"
).split()
V = {name: index for index, name in enumerate(_VALUE_OPS)}

REDUCE = {"max": 1, "min": 2, "sum": 3}


class MapOperand(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("segment", ctypes.c_int32), ("other", ctypes.c_double)]


class MapProgram(ctypes.Structure):
    _fields_ = [
        ("num_vars", ctypes.c_int32),
        ("num_reduced", ctypes.c_int32),
        ("num_dynamic", ctypes.c_int32),
        ("store_op", ctypes.c_int32),
        ("extents", ctypes.c_int64 * MAX_VARS),
        ("num_operands", ctypes.c_int32),
        ("output", ctypes.c_int32),
        ("operands", MapOperand * MAX_OPERANDS),
        ("num_segments", ctypes.c_int32),
        ("segment_begin", ctypes.c_int32 * MAX_SEGMENTS),
        ("index_code", ctypes.c_int32 * MAX_INDEX_CODE),
        ("index_constants", ctypes.c_int64 * MAX_INDEX_CONSTANTS),
        ("value_code_length", ctypes.c_int32),
        ("reduce_split", ctypes.c_int32),
        ("reduce_op", ctypes.c_int32),
        ("reduce_dtype", ctypes.c_int32),
        ("value_code", ctypes.c_int32 * MAX_VALUE_CODE),
        ("value_constants", ctypes.c_double * MAX_VALUE_CONSTANTS),
        ("num_phases", ctypes.c_int32),
        ("num_grid", ctypes.c_int32),
        ("phase_end", ctypes.c_int32 * MAX_PHASES),
        ("phase_op", ctypes.c_int32 * MAX_PHASES),
        ("phase_dtype", ctypes.c_int32 * MAX_PHASES),
    ]


# ---- types of values -----------------------------------------------------------

_FLOATS = ("fp16", "bf16", "fp32", "fp64")
_INT_RANK = {"bool": 0, "i8": 1, "u8": 1, "i16": 2, "u16": 2, "i32": 3, "u32": 3, "i64": 4, "u64": 4}
_LITERAL_INT, _LITERAL_FLOAT = "int literal", "float literal"


def _promote(a, b, division=False):
    """Result type of an arithmetic operation (Triton's rules for the generated code)."""
    literals = (_LITERAL_INT, _LITERAL_FLOAT)
    if a in literals and b in literals:
        return _LITERAL_FLOAT if _LITERAL_FLOAT in (a, b) or division else _LITERAL_INT
    if a in literals or b in literals:
        literal, other = (a, b) if a in literals else (b, a)
        if other in _FLOATS:
            return other
        return "fp32" if literal == _LITERAL_FLOAT or division else other
    if a in _FLOATS and b in _FLOATS:
        if a == b:
            return a
        if {a, b} == {"fp16", "bf16"}:
            return "fp32"
        return max(a, b, key=_FLOATS.index) if "fp64" in (a, b) or "fp32" in (a, b) else "fp32"
    if a in _FLOATS or b in _FLOATS:
        return a if a in _FLOATS else b
    if division:
        return "fp32"
    return a if _INT_RANK[a] >= _INT_RANK[b] else b


def _needs_rounding(dtype):
    return dtype in ("fp16", "bf16", "fp32") or dtype in _INT_RANK and dtype != "bool"


def operand_param(lowering, slot):
    return lowering.operands[slot][0]


# ---- the application: which programs are tile maps ----------------------------------

_BINARY = {
    "add": "ADD", "sub": "SUB", "mul": "MUL", "div": "DIV", "floordiv": "FLOORDIV", "mod": "MOD", "pow": "POW",
    "maximum": "MAX", "minimum": "MIN", "libdevice.pow": "POW",
}
_COMPARE = {"lt": "LT", "le": "LE", "gt": "GT", "ge": "GE", "eq": "EQ", "ne": "NE"}
_LOGICAL = {"and": "AND", "or": "OR"}
_UNARY_SAME = {"neg": "NEG", "abs": "ABS", "floor": "FLOOR", "ceil": "CEIL", "libdevice.floor": "FLOOR", "libdevice.ceil": "CEIL"}
_UNARY_FLOAT = {
    "exp": "EXP", "exp2": "EXP2", "log": "LOG", "log2": "LOG2", "sqrt": "SQRT", "rsqrt": "RSQRT", "sigmoid": "SIGMOID",
    "libdevice.tanh": "TANH", "libdevice.sin": "SIN", "libdevice.cos": "COS", "libdevice.exp": "EXP", "libdevice.log": "LOG",
    "libdevice.sqrt": "SQRT", "libdevice.rsqrt": "RSQRT", "sin": "SIN", "cos": "COS",
}


def _kwargs(node):
    positional, named = [], {}
    for arg in node.args:
        if isinstance(arg, Node) and arg.op == "kwarg":
            named[arg.args[0]] = arg.args[1]
        else:
            positional.append(arg)
    return positional, named


class _RawOperand:
    """A whole tensor addressed by computed indices (``x.source[i, j]``) or by a computed
    element offset (a raw pointer): ``terms`` lists (dynamic variable, stride, size or None)."""

    empty = False

    def __init__(self, tensor):
        self.tensor = tensor
        self.terms = []


def _affine_names(expr):
    """The index variables an affine index expression depends on."""
    names = set()
    for atom, coef in expr.terms.items():
        if coef == 0:
            continue
        if atom[0] == "var":
            names.add(atom[1])
        else:
            names |= _affine_names(Affine.from_key(atom[1]))
    return names


def _split_pointer(expr):
    """``x.source.data_ptr() + offsets`` -> (parameter of x, offsets in elements)."""
    found = []

    def strip(item):
        if isinstance(item, Node) and item.op == "data_ptr":
            found.append(item.args[0].param)
            return None
        if isinstance(item, Node) and item.op == "add":
            a, b = strip(item.args[0]), strip(item.args[1])
            if a is None or b is None:
                return b if a is None else a
            return Node("add", a, b)
        return item

    rest = strip(expr)
    if len(found) != 1:
        raise UnsupportedProgram("A pointer must be `tensor.source.data_ptr()` plus element offsets.")
    return found[0], 0 if rest is None else rest


_REDUCTIONS = ("max", "min", "sum")


def _first_tile_ref(value):
    """The first tile a value is built from outside of reductions: it fixes the shape of a store
    that goes through computed indices or a pointer."""
    if isinstance(value, Node):
        if value.op in _REDUCTIONS:
            return None
        if value.op in ("load", "offsets") and isinstance(value.args[0], TensorRef):
            return value.args[0]
        for arg in value.args:
            found = _first_tile_ref(arg)
            if found is not None:
                return found
    elif isinstance(value, (tuple, list)):
        for item in value:
            found = _first_tile_ref(item)
            if found is not None:
                return found
    return None


class _Lowering:
    """One store of one call: collects operands, index segments and value code."""

    def __init__(self, types, args, env, dtype_tag, tile_mode=False, scalar_dtypes=None):
        self.types, self.args, self.env, self.dtype_tag = types, args, env, dtype_tag
        # packaged kernels: a scalar has the element type it was declared with, whatever Python number
        # stands in for it (the reference's AOT signature, src/ninetoothed/aot.py:234-283)
        self.scalar_dtypes = scalar_dtypes or {}
        # tile mode: whole-tile reductions become phases whose results the expression may use on
        # every element of the tile; `phases` holds (operation, accumulate type, term code)
        self.tile_mode = tile_mode
        self.phases = []
        self.phase_of = {}        # digest of a reduction -> (phase, type of its term, type it accumulates in)
        self.tile_axis = None     # axis of the tile the phases reduce over (None: the whole tile)
        self.axis_subscript_seen = False
        self.operands = []        # (param, Operand)
        self.operand_slot = {}    # param -> slot
        self.var_extent = []      # shared variables: grid dims first, then output tile dims, then reduced dims
        self.grid = None          # list of variable ids of the launch grid
        self.segments = []        # (operand slot, kind, dim)
        self.segment_slot = {}
        self.value_code = []
        self.constants = []
        self.reduce = None        # (op name, accumulate dtype)
        self.reduce_split = None
        self.num_reduced = 0
        self.bindings = {}        # operand slot -> {operand variable name: shared variable id}
        self.scalar_slots = []    # (constant index, parameter position): refreshed at every launch
        self.symbolic_constants = {}  # constant index -> size expression (packaging only)
        self.reduced_vars = []
        self.dynamic_vars = []    # variables that take their value from the data (level indices)
        self.levels_used = {}     # param -> level its tiles are taken from
        self.jagged = {}          # operand slot -> (variable of the sequence start, variable of its end)

    # -- variables ---------------------------------------------------------
    def new_var(self, extent):
        self.var_extent.append(integer(extent))
        return len(self.var_extent) - 1

    def operand(self, param, level=1):
        if self.levels_used.setdefault(param, level) != level:
            raise UnsupportedProgram("A tensor is used at two different levels.")
        if param in self.operand_slot:
            return self.operand_slot[param]
        tensor = self.types[param]
        operand = Operand(tensor, self.env)
        if len(operand.names) > level + 1:
            raise UnsupportedProgram(f"`{tensor.source.name}` has a level below the tiles the application uses.")
        if len(operand.names) < level:
            raise UnsupportedProgram(f"`{tensor.source.name}` is indexed deeper than it is arranged.")
        grid_names = operand.names[0]
        if self.grid is None:
            self.grid = [self.new_var(operand.extents[name]) for name in grid_names]
        if len(grid_names) != len(self.grid):
            raise UnsupportedProgram("The arranged tensors disagree on the number of launch-grid dimensions.")
        binding = {}
        for name, var in zip(grid_names, self.grid):
            if operand.extents[name] != self.var_extent[var]:
                raise UnsupportedProgram(
                    f"`{tensor.source.name}` has {operand.extents[name]} tiles along a grid dimension where another tensor has {self.var_extent[var]}."
                )
            binding[name] = var
        slot = len(self.operands)
        if slot >= MAX_OPERANDS:
            raise UnsupportedProgram("Too many tensor operands for the element-wise executor.")
        self.operands.append((param, operand))
        self.operand_slot[param] = slot
        self.bindings[slot] = binding
        return slot

    def bind_tile(self, slot, dims):
        """Binds the operand's tile dimensions to the shared variables ``dims``."""
        _, operand = self.operands[slot]
        level = self.levels_used[operand_param(self, slot)]
        tile_names = operand.names[level] if len(operand.names) > level else []
        if len(tile_names) != len(dims):
            raise UnsupportedProgram(
                f"A tile of `{operand.tensor.source.name}` has {len(tile_names)} dimensions where the expression needs {len(dims)}."
            )
        binding = self.bindings[slot]
        for name, var in zip(tile_names, dims):
            extent = operand.extents[name]
            if self.var_extent[var] is None:
                self.var_extent[var] = extent
            elif self.var_extent[var] != extent:
                raise UnsupportedProgram(
                    f"Tiles of different shapes meet in one expression ({extent} against {self.var_extent[var]} elements); broadcasting tiles is not supported."
                )
            if binding.get(name, var) != var:
                raise UnsupportedProgram(f"`{operand.tensor.source.name}` is used with two different tile layouts.")
            binding[name] = var

    # -- value code -----------------------------------------------------------
    def emit(self, op, arg=0):
        self.value_code.append(V[op] | (arg << 8))

    def constant(self, value):
        if is_symbolic(value):  # a size of the call used as a value: its own slot, filled in per launch by packaged code
            self.constants.append(float(plain(value)))
            self.symbolic_constants[len(self.constants) - 1] = value
            return len(self.constants) - 1
        value = float(value)
        scalars = {index for index, _ in self.scalar_slots} | set(self.symbolic_constants)
        for index, known in enumerate(self.constants):
            if index not in scalars and (known == value or (known != known and value != value)):
                return index
        self.constants.append(value)
        return len(self.constants) - 1

    def round(self, dtype):
        if _needs_rounding(dtype):
            self.emit("ROUND", runtime.DATA_TYPE_INDEX[dtype])

    def segment(self, slot, kind, dim=None):
        key = (slot, kind, dim)
        if key not in self.segment_slot:
            self.segment_slot[key] = len(self.segments)
            self.segments.append(key)
        return self.segment_slot[key]

    def lower(self, value, dims, inside_reduction):
        """Emits code that leaves ``value`` on the stack; returns its type."""
        if isinstance(value, bool):
            self.emit("CONST", self.constant(1.0 if value else 0.0))
            return "bool"
        if isinstance(value, int):
            self.emit("CONST", self.constant(value))
            return _LITERAL_INT
        if isinstance(value, float):
            self.emit("CONST", self.constant(value))
            return _LITERAL_FLOAT
        if isinstance(value, ScalarParam):
            arg = self.args[value.param]
            self.constants.append(float(arg))  # a slot of its own: call-time scalars are refreshed per launch
            self.scalar_slots.append((len(self.constants) - 1, value.param))
            self.emit("CONST", len(self.constants) - 1)
            if value.param in self.scalar_dtypes:
                self.round(self.scalar_dtypes[value.param])
                return self.scalar_dtypes[value.param]
            if value.constexpr:
                return "bool" if isinstance(arg, bool) else _LITERAL_INT if isinstance(arg, int) else _LITERAL_FLOAT
            if isinstance(arg, bool):
                return "bool"
            if isinstance(arg, int):
                return "i32" if -(2**31) <= arg < 2**31 else "i64"
            self.round("fp32")
            return "fp32"
        if isinstance(value, (SourceDim, SourceStride)):
            source = self.types[value.param].source
            name = source.size_string(value.dim) if isinstance(value, SourceDim) else source.stride_string(value.dim)
            self.emit("CONST", self.constant(integer(self.env[name])))
            return _LITERAL_INT
        if isinstance(value, Dim):  # `x.shape[d]` of a level: a call-time integer
            level = self.types[value.param].levels()[value.level]
            self.emit("CONST", self.constant(integer(evaluate(level.shape[value.dim], self.env))))
            return _LITERAL_INT
        if not isinstance(value, Node):
            raise UnsupportedProgram(f"A value of type `{type(value).__name__}` cannot be stored by the element-wise executor.")

        op = value.op
        if op == "load" and not isinstance(value.args[0], TensorRef):  # `ntl.load(pointer)`
            positional, named = _kwargs(value)
            if len(positional) != 1 or named:
                raise UnsupportedProgram("`ntl.load` of a pointer takes no mask here; index `tensor.source[...]` for a masked load.")
            param, offset = _split_pointer(positional[0])
            slot = self.raw_access(param, None, dims, inside_reduction, element_offset=offset)
            self.emit("LOAD", slot)
            return self.dtype_tag(param)
        if op == "source_at":
            source, indices = value.args
            slot = self.raw_access(source.param, indices, dims, inside_reduction)
            self.emit("LOAD", slot)
            return self.dtype_tag(source.param)
        if op == "index":
            return self.lower_oriented_offsets(value, dims, inside_reduction)
        if op == "load":
            ref = value.args[0]
            self._check_ref(ref)
            if self.reduce is not None and not inside_reduction:
                raise UnsupportedProgram("Tiles may only be loaded below the reduction of the expression.")
            slot = self.bind_ref(ref, dims, inside_reduction)
            self.emit("LOAD", slot)
            return self.dtype_tag(ref.param)
        if op == "offsets":
            ref, dim = value.args
            self._check_ref(ref)
            slot = self.bind_ref(ref, dims, inside_reduction)
            self.emit("OFFSET", self.segment(slot, "offsets", dim))
            return "i64" if dim is None else "i32"
        if op in _BINARY or op in _COMPARE or op in _LOGICAL:
            positional, _ = _kwargs(value)
            if len(positional) != 2:
                raise UnsupportedProgram(f"`{op}` takes two operands.")
            # a Python literal (or a constexpr scalar) takes the type of the tile it meets
            # before the operation, as a constant of that type would
            literals = (_LITERAL_INT, _LITERAL_FLOAT)
            a = self.lower(positional[0], dims, inside_reduction)
            mark = len(self.value_code)
            b = self.lower(positional[1], dims, inside_reduction)
            if a in literals and b not in literals and _needs_rounding(_promote(a, b)):
                self.value_code.insert(mark, V["ROUND"] | (runtime.DATA_TYPE_INDEX[_promote(a, b)] << 8))
                if self.reduce_split is not None and self.reduce_split >= mark:
                    self.reduce_split += 1
            elif b in literals and a not in literals and _needs_rounding(_promote(a, b)):
                self.emit("ROUND", runtime.DATA_TYPE_INDEX[_promote(a, b)])
            if op in _COMPARE:
                self.emit(_COMPARE[op])
                return "bool"
            if op in _LOGICAL:
                self.emit(_LOGICAL[op])
                return "bool"
            result = _promote(a, b, division=op == "div")
            if op in ("pow", "libdevice.pow") and result not in _FLOATS:
                result = "fp32"
            self.emit(_BINARY[op])
            self.round(result)
            return result
        if op in _UNARY_SAME or op in _UNARY_FLOAT:
            positional, _ = _kwargs(value)
            a = self.lower(positional[0], dims, inside_reduction)
            if op in _UNARY_FLOAT:
                if a not in _FLOATS:
                    a = "fp32"
                self.emit(_UNARY_FLOAT[op])
                self.round(a)
            else:
                self.emit(_UNARY_SAME[op])
            return a
        if op == "pos":
            return self.lower(value.args[0], dims, inside_reduction)
        if op == "not":
            self.lower(value.args[0], dims, inside_reduction)
            self.emit("NOT")
            return "bool"
        if op == "where":
            positional, _ = _kwargs(value)
            if len(positional) != 3:
                raise UnsupportedProgram("`where` takes a condition and two values.")
            self.lower(positional[0], dims, inside_reduction)
            a = self.lower(positional[1], dims, inside_reduction)
            b = self.lower(positional[2], dims, inside_reduction)
            self.emit("WHERE")
            result = _promote(a, b)
            self.round(result)
            return result
        if op == "cast":
            source, target = value.args
            self.lower(source, dims, inside_reduction)
            if isinstance(target, ElementType):
                target = self.dtype_tag(target.param)
            if not isinstance(target, str) or target not in runtime.DATA_TYPE_INDEX:
                raise UnsupportedProgram(f"Cannot cast to `{target!r}`.")
            self.emit("ROUND", runtime.DATA_TYPE_INDEX[target])
            return target
        if op == "rand":
            positional, _ = _kwargs(value)
            if len(positional) != 2:
                raise UnsupportedProgram("`rand` takes a seed and offsets.")
            self.lower(positional[0], dims, inside_reduction)
            self.lower(positional[1], dims, inside_reduction)
            self.emit("RAND")
            return "fp32"
        if op in REDUCE and self.tile_mode:
            positional, named = _kwargs(value)
            axis = named.get("axis", positional[1] if len(positional) > 1 else None)
            if self._tile_rank(positional[0]) != len(dims):
                raise UnsupportedProgram("A reduction whose result is used on a tile must run over tiles of that tile's shape.")
            # every reduction of the expression runs over the same part of the tile: all of it, or one
            # axis (then the other tile dimensions enumerate "rows", each reduced on its own, and the
            # result is laid back over the tile with a `None` subscript at that axis)
            if axis is not None:
                if not isinstance(axis, int) or not -len(dims) <= axis < len(dims):
                    raise UnsupportedProgram("The reduction axis must be an integer constant within the tile's dimensions.")
                axis %= len(dims)
                if not self.axis_subscript_seen:
                    raise UnsupportedProgram("Subscript the result of an axis reduction with `None` at that axis to use it on the tile.")
                self.axis_subscript_seen = False
            if self.phases and self.tile_axis != axis:
                raise UnsupportedProgram("All reductions of one stored expression must run over the same axis.")
            self.tile_axis = axis
            if value.digest in self.phase_of:  # the same reduction used again: one phase serves every use
                k, term, accumulate = self.phase_of[value.digest]
                self.emit("REDUCED", k)
                if accumulate != term:
                    self.round(term)
                return term
            outer_code, self.value_code = self.value_code, []
            try:
                term = self.lower(positional[0], dims, inside_reduction)
                code = self.value_code
            finally:
                self.value_code = outer_code
            if term in (_LITERAL_INT, _LITERAL_FLOAT):
                raise UnsupportedProgram("A reduction needs a tile operand.")
            if len(self.phases) >= MAX_PHASES:
                raise UnsupportedProgram("Too many reductions in one stored expression.")
            accumulate = "fp32" if op == "sum" and term in ("fp16", "bf16") else term
            self.phases.append((op, accumulate, code))
            self.phase_of[value.digest] = (len(self.phases) - 1, term, accumulate)
            self.emit("REDUCED", len(self.phases) - 1)
            if accumulate != term:
                self.round(term)
            return term
        if op in REDUCE:
            if self.reduce is not None or inside_reduction:
                raise UnsupportedProgram("Only one reduction per stored expression is supported.")
            positional, named = _kwargs(value)
            axis = named.get("axis", positional[1] if len(positional) > 1 else None)
            if axis is not None and not isinstance(axis, int):
                raise UnsupportedProgram("The reduction axis must be an integer constant.")
            if self.value_code:
                raise UnsupportedProgram("A reduction must be the innermost tile operation of the stored expression.")
            if axis is None:
                if any(self.var_extent[var] != 1 for var in dims):
                    raise UnsupportedProgram("A full reduction yields a scalar; the stored tile has more than one element.")
                rank = self._tile_rank(positional[0])
                inner = [self.new_var_deferred() for _ in range(rank)]
                reduced = list(inner)
            else:
                rank = len(dims) + 1
                axis %= rank
                fresh = self.new_var_deferred()
                inner = list(dims[:axis]) + [fresh] + list(dims[axis:])
                reduced = [fresh]
            self.reduced_vars = reduced
            self.reduce = (op, None)
            term = self.lower(positional[0], inner, True)
            accumulate = "fp32" if op == "sum" and term in ("fp16", "bf16") else term
            if term in (_LITERAL_INT, _LITERAL_FLOAT):
                raise UnsupportedProgram("A reduction needs a tile operand.")
            self.reduce = (op, accumulate)
            self.reduce_split = len(self.value_code)
            if accumulate != term:
                self.round(term)
            return term
        raise UnsupportedProgram(f"`{op}` is not an element-wise operation this build can execute.")

    def lower_oriented_offsets(self, value, dims, inside_reduction):
        """``x.offsets(d)[:, None]``: the indices along source dimension ``d`` laid along one
        dimension of the tile (src/ninetoothed/generation.py:212-230).  Values are computed per
        tile element here, so this is the plain ``offsets(d)`` provided that index really only
        varies along the dimension the subscript names."""
        base, keys = value.args
        if not all(key is None or key == slice(None) for key in keys):
            raise UnsupportedProgram("Tiles and `.offsets(dim)` can only be subscripted with `:` and `None`.")
        if isinstance(base, Node) and base.op in REDUCE and self.tile_mode:
            # `ntl.max(x, axis=1)[:, None]`: one value per row of the tile, laid back over the tile
            positional, named = _kwargs(base)
            axis = named.get("axis", positional[1] if len(positional) > 1 else None)
            if not isinstance(axis, int) or len(keys) != len(dims):
                raise UnsupportedProgram("Only the result of an axis reduction of the tile can be subscripted with `None`.")
            expected = tuple(None if position == axis % len(dims) else slice(None) for position in range(len(dims)))
            if tuple(keys) != expected:
                raise UnsupportedProgram("The `None` of the subscript must stand at the reduced axis.")
            self.axis_subscript_seen = True
            return self.lower(base, dims, inside_reduction)
        if isinstance(base, Node) and base.op == "load" and isinstance(base.args[0], TensorRef):
            # `bias[None, :]`: a tile of lower rank laid along the dimensions the `:` entries name;
            # every element of the result reads the element of the tile at those coordinates
            if len(keys) != len(dims):
                raise UnsupportedProgram("A broadcast subscript needs as many entries as the expression's tiles have dimensions.")
            return self.lower(base, [dim for dim, key in zip(dims, keys) if key is not None], inside_reduction)
        plain = isinstance(base, Node) and base.op == "offsets" and base.args[1] is not None
        if not plain:
            raise UnsupportedProgram("Only tiles and `.offsets(dim)` can be subscripted with `:` and `None`.")
        along = [position for position, key in enumerate(keys) if key is not None]
        if len(along) != 1 or len(keys) != len(dims):
            raise UnsupportedProgram("A subscript of `.offsets(dim)` needs one `:` and as many entries as the tile has dimensions.")
        ref, dim = base.args
        self._check_ref(ref)
        slot = self.bind_ref(ref, dims, inside_reduction)
        _, operand = self.operands[slot]
        binding = self.bindings[slot]
        allowed = {dims[along[0]]} | set(self.grid) | set(self.dynamic_vars)
        for name in _affine_names(operand.indices[dim]):
            if binding.get(name) not in allowed and operand.extents.get(name, 1) != 1:
                raise UnsupportedProgram("`.offsets(dim)` varies along another tile dimension than the one its subscript names.")
        self.emit("OFFSET", self.segment(slot, "offsets", dim))
        return "i32"

    def raw_access(self, param, indices, dims, inside_reduction, element_offset=None):
        """Registers an operand addressed by computed values; emits the code that computes them."""
        slot = len(self.operands)
        if slot >= MAX_OPERANDS:
            raise UnsupportedProgram("Too many tensor operands for the element-wise executor.")
        tensor = None if isinstance(param, tuple) else self.types[param]  # (position, "offsets"): sequence offsets of a jagged tensor
        if tensor is not None and tensor.ndim == 0 and not hasattr(tensor.dtype, "ndim"):
            raise UnsupportedProgram("Scalars have no elements to address.")
        if tensor is not None and tensor.source.jagged_dim is not None:
            raise UnsupportedProgram("Jagged tensors cannot be addressed by computed indices or pointers.")
        raw = _RawOperand(tensor)
        self.operands.append((param, raw))
        self.bindings[slot] = {}

        def dynamic(value, size):
            var = self.new_var(max(integer(size), 1) if size is not None else 1)
            self.dynamic_vars.append(var)
            self.lower(value, dims, inside_reduction)
            self.emit("SETVAR", var)
            return var

        if element_offset is not None:
            raw.terms.append((dynamic(element_offset, None), 1, None))
            return slot
        source = tensor.source
        if len(indices) != source.ndim:
            raise UnsupportedProgram("A source tensor needs one index per dimension.")
        for dim, index in enumerate(indices):
            size = integer(self.env[source.size_string(dim)])
            raw.terms.append((dynamic(index, size), integer(self.env[source.stride_string(dim)]), size))
        return slot

    def new_var_deferred(self):
        self.var_extent.append(None)
        return len(self.var_extent) - 1

    def _tile_rank(self, value):
        ranks = set()

        def visit(item):
            if isinstance(item, Node):
                if item.op == "load" and isinstance(item.args[0], TensorRef):
                    ref = item.args[0]
                    tensor = self.types[ref.param]
                    ranks.add(tensor.dtype.ndim if hasattr(tensor.dtype, "ndim") else 0)
                for arg in item.args:
                    visit(arg)
            elif isinstance(item, (tuple, list)):
                for arg in item:
                    visit(arg)

        visit(value)
        if len(ranks) != 1:
            raise UnsupportedProgram("The operand of a full reduction must be built from tiles of one rank.")
        return ranks.pop()

    def _check_ref(self, ref):
        if not isinstance(ref, TensorRef) or ref.level not in (1, 2) or not ref.is_tile:
            raise UnsupportedProgram("Only whole tiles one or two levels below the launch grid can be used by the element-wise executor.")

    def bind_ref(self, ref, dims, inside_reduction):
        """Registers the operand of ``ref``, binds its tile to ``dims`` and, for a tile taken
        from a middle level (``tensor[i, j]``), emits the code that computes the level indices."""
        slot = self.operand(ref.param, ref.level)
        self.bind_tile(slot, dims)
        if self.types[ref.param].source.jagged_dim is not None and slot not in self.jagged:
            self.bind_sequence(slot, ref, dims, inside_reduction)
        if ref.level == 2:
            _, operand = self.operands[slot]
            names = operand.names[1]
            if len(ref.indices) != len(names):
                raise UnsupportedProgram("A level must be indexed with one index per dimension.")
            binding = self.bindings[slot]
            for name, index in zip(names, ref.indices):
                if name in binding:
                    raise UnsupportedProgram("A tensor may be indexed at a middle level only once per program.")
                var = self.new_var(operand.extents[name])
                self.dynamic_vars.append(var)
                binding[name] = var
                # the index is a scalar: a constant, a call-time scalar or a one-element tile
                rank = self._tile_rank(index) if isinstance(index, Node) and self._has_load(index) else 0
                unit = [self.new_var(1) for _ in range(rank)]
                self.lower(index, unit, inside_reduction)
                self.emit("SETVAR", var)
        return slot

    def bind_sequence(self, slot, ref, dims, inside_reduction):
        """A jagged tensor: loads where the batch entry's sequence starts and ends in the values
        (``offsets[batch]``, ``offsets[batch + 1]``; src/ninetoothed/generation.py:686-704) into
        two variables the index program of the operand uses."""
        if ref.level != 1:
            raise UnsupportedProgram("Jagged tensors are supported with tiles directly below the launch grid.")
        start, end = self.new_var(1), self.new_var(1)
        self.dynamic_vars += [start, end]
        self.jagged[slot] = (start, end)
        batch = Node("offsets", ref, 0)
        for var, position in ((start, batch), (end, Node("add", batch, 1))):
            bounds = self.raw_access((ref.param, "offsets"), None, dims, inside_reduction, element_offset=position)
            self.emit("LOAD", bounds)
            self.emit("SETVAR", var)

    def _has_load(self, value):
        if isinstance(value, Node):
            return (value.op == "load" and isinstance(value.args[0], TensorRef)) or any(self._has_load(arg) for arg in value.args)
        if isinstance(value, (tuple, list)):
            return any(self._has_load(item) for item in value)
        return False

    # -- index code ----------------------------------------------------------------
    def index_program(self, order):
        """Returns (code words, constants, segment begins) for all segments, with the
        shared variables renumbered by ``order`` (old id -> new id)."""
        code, constants, begins = [], [], []

        def const(value):
            value = integer(value)
            for index, known in enumerate(constants):
                if same(known, value):
                    return index
            constants.append(value)
            return len(constants) - 1

        def emit_affine(expr, binding):
            code.append(I_CONST | (const(expr.const) << 8))
            for atom, coef in sorted(expr.terms.items(), key=repr):
                if atom[0] == "var":
                    if atom[1] not in binding:
                        raise UnsupportedProgram(f"Index variable `{atom[1]}` is not part of the iteration space.")
                    code.append(I_VAR | (order[binding[atom[1]]] << 8))
                else:
                    emit_affine(Affine.from_key(atom[1]), binding)
                    code.append((I_DIVC if atom[0] == "div" else I_MODC) | (const(atom[2]) << 8))
                if is_symbolic(coef) or coef != 1:
                    code.append(I_MULC | (const(coef) << 8))
                code.append(I_ADD)

        def emit_sequence_start(slot, operand):
            if slot in self.jagged:
                source = operand.tensor.source
                code.append(I_VAR | (order[self.jagged[slot][0]] << 8))
                code.append(I_MULC | (const(integer(self.env[source.stride_string(source.jagged_dim)])) << 8))
                code.append(I_ADD)

        for slot, kind, dim in self.segments:
            _, operand = self.operands[slot]
            binding = self.bindings[slot]
            begins.append(len(code))
            if kind == "raw":
                for var, _, size in operand.terms:
                    if size is not None:
                        code.append(I_VAR | (order[var] << 8))
                        code.append(I_CHECK | (const(size) << 8))
                code.append(I_CONST | (const(0) << 8))
                for var, stride, _ in operand.terms:
                    code.append(I_VAR | (order[var] << 8))
                    if is_symbolic(stride) or stride != 1:
                        code.append(I_MULC | (const(stride) << 8))
                    code.append(I_ADD)
            elif kind == "access":
                # indices that come from the data are range-checked: an element outside its level
                # is treated like a masked one (the reference would access out of bounds)
                for name, var in binding.items():
                    if var in self.dynamic_vars:
                        code.append(I_VAR | (order[var] << 8))
                        code.append(I_CHECK | (const(operand.extents[name]) << 8))
                for index, size in operand.constraints:
                    emit_affine(index, binding)
                    code.append(I_CHECK | (const(size) << 8))
                if slot in self.jagged:
                    # inside the sequence: 0 <= end - 1 - start - index (its lower bound is the tile mask above,
                    # or holds by construction); the values are then addressed from the sequence's start
                    start, end = self.jagged[slot]
                    jagged_dim = operand.tensor.source.jagged_dim
                    code.append(I_VAR | (order[end] << 8))
                    code.append(I_CONST | (const(-1) << 8))
                    code.append(I_ADD)
                    for term in (None, operand.indices[jagged_dim]):
                        if term is None:
                            code.append(I_VAR | (order[start] << 8))
                        else:
                            emit_affine(term, binding)
                        code.append(I_MULC | (const(-1) << 8))
                        code.append(I_ADD)
                    code.append(I_CHECK | (const(1 << 62) << 8))
                    emit_affine(operand.indices[jagged_dim], binding)
                    code.append(I_CHECK | (const(1 << 62) << 8))
                emit_affine(operand.offset(), binding)
                emit_sequence_start(slot, operand)
            elif dim is None:
                emit_affine(operand.offset(), binding)
                emit_sequence_start(slot, operand)
            else:
                emit_affine(operand.indices[dim], binding)
            code.append(I_END)
        return code, constants, begins


def _as_element(value, tag):
    """``value`` as an element of type ``tag`` holds it (a masked load yields a tile of the
    tensor's type, so `other` is rounded like any constant of that type)."""
    import struct

    if value != value or value in (float("inf"), float("-inf")):
        return value
    if tag == "fp16":
        import numpy as np

        with np.errstate(over="ignore"):
            return float(np.float16(value))
    if tag == "bf16":
        bits = struct.unpack("<I", struct.pack("<f", value))[0]
        bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
        return struct.unpack("<f", struct.pack("<I", bits & 0xFFFFFFFF))[0]
    if tag == "fp32":
        return struct.unpack("<f", struct.pack("<f", value))[0]
    if tag == "fp64":
        return float(value)
    return float(int(value))


def _other_value(tensor):
    if tensor is None:
        return 0.0
    other = tensor.source.other
    return 0.0 if other is None else float(other)


def _has_whole_tile_reduction(value):
    """Whether the expression reduces whole tiles, or uses an axis reduction on the tile (`m[:, None]`)."""
    if isinstance(value, Node):
        if value.op in REDUCE:
            positional, named = _kwargs(value)
            if named.get("axis", positional[1] if len(positional) > 1 else None) is None:
                return True
        if value.op == "index" and isinstance(value.args[0], Node) and value.args[0].op in REDUCE:
            return True
        return any(_has_whole_tile_reduction(arg) for arg in value.args)
    if isinstance(value, (tuple, list)):
        return any(_has_whole_tile_reduction(item) for item in value)
    return False


def build(program_store, types, args, env, dtype_tag, data_ptr, scalar_dtypes=None):
    """Builds the :class:`MapProgram` of one store for one call.  Returns
    ``None`` when the launch is empty.

    A reduction is first tried as the innermost operation of the expression (one result per
    output element); when the expression does not have that form but reduces whole tiles, the
    program is built in tile mode (reductions as phases of a workgroup that owns the tile)."""
    try:
        return _build(program_store, types, args, env, dtype_tag, data_ptr, False, scalar_dtypes)
    except UnsupportedProgram:
        if not isinstance(program_store[0], TensorRef) or not _has_whole_tile_reduction(program_store[1]):
            raise
        return _build(program_store, types, args, env, dtype_tag, data_ptr, True, scalar_dtypes)


def _build(program_store, types, args, env, dtype_tag, data_ptr, tile_mode, scalar_dtypes=None):
    ref, value = program_store
    lowering = _Lowering(types, args, env, dtype_tag, tile_mode, scalar_dtypes)
    store_op = 0
    if isinstance(ref, TensorRef):
        lowering._check_ref(ref)
        out_slot = order_slot = lowering.operand(ref.param, ref.level)
        _, out_operand = lowering.operands[out_slot]
        tile_names = out_operand.names[ref.level] if len(out_operand.names) > ref.level else []
        out_dims = [lowering.new_var(out_operand.extents[name]) for name in tile_names]
        lowering.bind_ref(ref, out_dims, False)
        result = lowering.lower(value, out_dims, False)
        out_dtype = dtype_tag(ref.param)
        if result != out_dtype:
            lowering.emit("ROUND", runtime.DATA_TYPE_INDEX[out_dtype])
    else:
        # a store through computed indices or a pointer: the first tile of the expression gives the shape
        anchor = _first_tile_ref((ref.args, value))
        order_slot, out_dims = None, []
        if anchor is not None:
            lowering._check_ref(anchor)
            order_slot = lowering.operand(anchor.param, anchor.level)
            _, anchor_operand = lowering.operands[order_slot]
            tile_names = anchor_operand.names[anchor.level] if len(anchor_operand.names) > anchor.level else []
            out_dims = [lowering.new_var(anchor_operand.extents[name]) for name in tile_names]
            lowering.bind_ref(anchor, out_dims, False)
        if ref.op == "source_at":
            out_param, indices, offset = ref.args[0].param, ref.args[1], None
        else:
            (out_param, offset), indices = _split_pointer(ref.args[0]), None
            store_op = 1 if ref.op == "pointer_atomic_add" else 0
        result = lowering.lower(value, out_dims, False)
        if lowering.grid is None:
            raise UnsupportedProgram("The stored value is not built from any arranged tensor.")
        out_dtype = dtype_tag(out_param)
        if result != out_dtype:
            lowering.emit("ROUND", runtime.DATA_TYPE_INDEX[out_dtype])
        out_slot = lowering.raw_access(out_param, indices, out_dims, False, element_offset=offset)
    if tile_mode:
        if lowering.dynamic_vars or lowering.reduce is not None or not lowering.phases or store_op != 0:
            raise UnsupportedProgram("Whole-tile reductions cannot be combined with data-dependent indices or atomic stores.")
        # phases first (in the order they were completed: a phase only uses earlier ones), then the stored expression
        final_code, lowering.value_code = lowering.value_code, []
        phase_ends = []
        for _, _, code in lowering.phases:
            lowering.value_code += code
            phase_ends.append(len(lowering.value_code))
        lowering.value_code += final_code
    if lowering.reduce is None:
        lowering.reduce_split = len(lowering.value_code)
    for slot, (_, operand) in enumerate(lowering.operands):
        lowering.segment(slot, "raw" if isinstance(operand, _RawOperand) else "access")
    if any(operand.empty for _, operand in lowering.operands):
        return None
    if any(extent is None for extent in lowering.var_extent):
        raise UnsupportedProgram("A reduced dimension is not covered by any tile.")

    # variable order: grid and output-tile variables enumerate the output elements
    # (the fastest one is chosen so that lanes walk the output contiguously), reduced ones follow
    reduced = list(lowering.reduced_vars)
    dynamic = list(lowering.dynamic_vars)
    outer = [v for v in range(len(lowering.var_extent)) if v not in reduced and v not in dynamic]
    stride_of = {}
    if order_slot is not None:
        offset = lowering.operands[order_slot][1].offset()
        for name, var in lowering.bindings[order_slot].items():
            stride_of[var] = abs(plain(offset.coef(name))) if offset.is_linear() else None
    if order_slot is not None and all(stride_of.get(v) is not None for v in outer):
        # (plain values: the order is a layout choice that no size of a call can make wrong)
        outer.sort(key=lambda v: (-(stride_of[v] or 1 << 62) if plain(lowering.var_extent[v]) > 1 else -(1 << 62), v))
    if tile_mode:  # the variables that enumerate tiles (or rows of tiles) first, then the reduced ones (fastest last, as sorted)
        reduced_over = set(out_dims) if lowering.tile_axis is None else {out_dims[lowering.tile_axis]}
        grid_vars = [v for v in outer if v not in reduced_over]
        outer = grid_vars + [v for v in outer if v in reduced_over]
    order = {old: new for new, old in enumerate(outer + reduced + dynamic)}
    # SETVAR words were emitted with provisional ids: renumber them like the index code
    for position, word in enumerate(lowering.value_code):
        if word & 0xFF == V["SETVAR"]:
            lowering.value_code[position] = V["SETVAR"] | (order[word >> 8] << 8)
    if len(order) > MAX_VARS:
        raise UnsupportedProgram("Too many index variables for the element-wise executor.")

    code, constants, begins = lowering.index_program(order)
    if len(code) > MAX_INDEX_CODE or len(constants) > MAX_INDEX_CONSTANTS or len(begins) > MAX_SEGMENTS:
        raise UnsupportedProgram("The index maps are too long for the element-wise executor.")
    if len(lowering.value_code) > MAX_VALUE_CODE or len(lowering.constants) > MAX_VALUE_CONSTANTS:
        raise UnsupportedProgram("The expression is too long for the element-wise executor.")

    program = MapProgram()
    patches = []  # (C lvalue inside the program, size expression): what packaged code recomputes per launch

    def number(field, value):
        if is_symbolic(value):
            patches.append((field, value))
        return plain(value)

    program.num_vars = len(outer) + len(reduced)
    program.num_reduced = len(reduced)
    program.num_dynamic = len(dynamic)
    for old, new in order.items():
        program.extents[new] = number(f"extents[{new}]", lowering.var_extent[old])
    program.store_op = store_op
    if tile_mode:
        program.num_phases = len(lowering.phases)
        program.num_grid = len(grid_vars)
        for k, (op, accumulate, _) in enumerate(lowering.phases):
            program.phase_end[k] = phase_ends[k]
            program.phase_op[k] = REDUCE[op]
            program.phase_dtype[k] = runtime.DATA_TYPE_INDEX[accumulate]
    program.num_operands = len(lowering.operands)
    program.output = out_slot
    for slot, (param, operand) in enumerate(lowering.operands):
        program.operands[slot].data = data_ptr(param)
        program.operands[slot].dtype = runtime.DATA_TYPE_INDEX[dtype_tag(param)]
        program.operands[slot].segment = lowering.segment_slot[(slot, "raw" if isinstance(operand, _RawOperand) else "access", None)]
        program.operands[slot].other = _as_element(_other_value(operand.tensor), dtype_tag(param))
    program.num_segments = len(begins)
    for index, begin in enumerate(begins):
        program.segment_begin[index] = begin
    for index, word in enumerate(code):
        program.index_code[index] = word
    for index, value_ in enumerate(constants):
        program.index_constants[index] = number(f"index_constants[{index}]", value_)
    program.value_code_length = len(lowering.value_code)
    program.reduce_split = lowering.reduce_split
    program.reduce_op = REDUCE[lowering.reduce[0]] if lowering.reduce else 0
    program.reduce_dtype = runtime.DATA_TYPE_INDEX[lowering.reduce[1]] if lowering.reduce else 0
    for index, word in enumerate(lowering.value_code):
        program.value_code[index] = word
    for index, value_ in enumerate(lowering.constants):
        program.value_constants[index] = value_
    for index, value_ in lowering.symbolic_constants.items():
        patches.append((f"value_constants[{index}]", value_))
    description = (
        f"{len(lowering.operands)} operands, {program.num_vars} index variables {[plain(lowering.var_extent[old]) for old in outer + reduced]}, "
        + (f"{len(dynamic)} data-dependent, " if dynamic else "")
        + 
        f"{len(code)} index words, {len(lowering.value_code)} value words"
        + (f", {lowering.reduce[0]} over {len(reduced)} dimension(s)" if lowering.reduce else "")
        + (f", {len(lowering.phases)} whole-tile reduction(s), one workgroup per tile" if tile_mode else "")
    )
    program.patches = patches
    return program, description, list(lowering.scalar_slots), [param for param, _ in lowering.operands]


def check_application(program):
    """Raises :class:`UnsupportedProgram` unless every store has the shape the
    executor handles (sizes are checked later, per call)."""

    for ref, value in program.stores:
        if isinstance(ref, Node) and ref.op in ("source_at", "pointer_store", "pointer_atomic_add"):
            _scan(ref.args)
            _scan(value)
            continue
        if not isinstance(ref, TensorRef) or ref.level not in (1, 2) or not ref.is_tile:
            raise UnsupportedProgram("Stores must assign whole tiles one or two levels below the launch grid.")
        _scan(ref.indices)
        _scan(value)


def _scan(value):
    if isinstance(value, Node):
        known = (
            set(_BINARY) | set(_COMPARE) | set(_LOGICAL) | set(_UNARY_SAME) | set(_UNARY_FLOAT) | set(REDUCE)
            | {"load", "offsets", "pos", "not", "where", "cast", "rand", "kwarg", "index", "source_at", "data_ptr"}
        )
        if value.op not in known:
            raise UnsupportedProgram(f"`{value.op}` is not an element-wise operation this build can execute.")
        for arg in value.args:
            _scan(arg)
    elif isinstance(value, (tuple, list)):
        for item in value:
            _scan(item)
    elif isinstance(value, TensorRef):
        if value.level not in (1, 2) or not value.is_tile:
            raise UnsupportedProgram("Only whole tiles one or two levels below the launch grid can be used by the element-wise executor.")
        _scan(value.indices)
