"""Turns an application (a Python function written against ``ntl``) into a
dataflow graph, without executing it.

The reference rewrites the application's AST into Triton source
(src/ninetoothed/generation.py:46-365: loads for tensor names, stores for
assignments to tensor parameters, compile-time resolution of ``.shape`` /
``.dtype`` / ``.source`` / ``.offsets(dim)``, and inlining of plain Python
helpers the application calls, src/ninetoothed/generation.py:884-1114).  This
module walks the same AST with the same conventions but builds a small
expression graph instead of text:

* a parameter name denotes the arranged tensor *below* the launch-grid level;
  subscripting moves down the hierarchy; using a tile in an expression loads it;
* assigning to a tensor parameter (or to a subscript of one) stores a tile;
* ``for i in range(n)`` becomes one ``loop`` node whose carried values are the
  names the body reassigns;
* ``if flag:`` on a call-time scalar becomes ``select`` nodes;
* helper calls are expanded in place, and a helper assigning to one of its
  parameters rebinds the caller's variable.

Every node has a structural digest; two applications with the same dataflow
have the same :attr:`Program.digest` whatever their variable names are.
"""

import ast
import builtins
import hashlib
import inspect
import textwrap
import types

from ninetoothed_amd import language
from ninetoothed_amd.tensor import Tensor


class TracingError(Exception):
    """The application uses something the tracer has no meaning for."""


# ---- values -----------------------------------------------------------------


class Node:
    """An operation in the dataflow graph."""

    __slots__ = ("op", "args", "_digest")

    def __init__(self, op, *args):
        self.op = op
        self.args = args
        self._digest = None

    @property
    def digest(self):
        if self._digest is None:
            parts = [_digest_of(arg) for arg in self.args]
            if self.op in _COMMUTATIVE:
                parts.sort()
            text = self.op + "(" + ",".join(parts) + ")"
            self._digest = hashlib.sha1(text.encode()).hexdigest()[:20]
        return self._digest

    def __repr__(self):
        return f"{self.op}({', '.join(map(_short, self.args))})"


_COMMUTATIVE = {"add", "mul", "maximum", "minimum", "and", "or", "eq", "ne"}


class TensorRef:
    """A parameter's arranged tensor at some level, partially indexed."""

    __slots__ = ("param", "tensor", "level", "indices")

    def __init__(self, param, tensor, level, indices=()):
        self.param = param      # position among the application's parameters
        self.tensor = tensor    # the level (a symbolic Tensor) this ref points at
        self.level = level      # 1 = just below the launch grid
        self.indices = indices  # indices applied to levels 1 .. level-1, flattened

    @property
    def is_tile(self):
        return not isinstance(self.tensor.dtype, Tensor)


class _Element:
    """The level below the grid of an untiled tensor: one element, no dimensions."""

    ndim = 0
    shape = ()
    dtype = None


_ELEMENT = _Element()


class ScalarParam:
    """A zero-dimensional tensor parameter (a call-time scalar)."""

    __slots__ = ("param", "constexpr")

    def __init__(self, param, constexpr):
        self.param = param
        self.constexpr = constexpr


class Dim:
    """The size of one dimension of a level of a parameter's arranged tensor."""

    __slots__ = ("param", "level", "dim")

    def __init__(self, param, level, dim):
        self.param, self.level, self.dim = param, level, dim


class SourceRef:
    __slots__ = ("param",)

    def __init__(self, param):
        self.param = param


class SourceDim:
    """The size of one dimension of a parameter's source tensor."""

    __slots__ = ("param", "dim")

    def __init__(self, param, dim):
        self.param, self.dim = param, dim


class SourceStride:
    """The stride (in elements) of one dimension of a parameter's source tensor."""

    __slots__ = ("param", "dim")

    def __init__(self, param, dim):
        self.param, self.dim = param, dim


class ElementType:
    """The element type of a parameter's source tensor."""

    __slots__ = ("param",)

    def __init__(self, param):
        self.param = param


class LoopVar:
    __slots__ = ("loop",)

    def __init__(self, loop):
        self.loop = loop


class Carried:
    """The value a loop-carried name has at the start of an iteration."""

    __slots__ = ("loop", "slot")

    def __init__(self, loop, slot):
        self.loop, self.slot = loop, slot


class _Range:
    __slots__ = ("extent",)

    def __init__(self, extent):
        self.extent = extent


def _digest_of(value):
    if isinstance(value, Node):
        return value.digest
    if isinstance(value, TensorRef):
        return f"ref[{value.param},{value.level}," + ",".join(map(_digest_of, value.indices)) + "]"
    if isinstance(value, ScalarParam):
        return f"scalar[{value.param}]"
    if isinstance(value, Dim):
        return f"dim[{value.param},{value.level},{value.dim}]"
    if isinstance(value, SourceDim):
        return f"srcdim[{value.param},{value.dim}]"
    if isinstance(value, SourceStride):
        return f"srcstride[{value.param},{value.dim}]"
    if isinstance(value, SourceRef):
        return f"source[{value.param}]"
    if isinstance(value, ElementType):
        return f"elemtype[{value.param}]"
    if isinstance(value, LoopVar):
        return f"loopvar[{value.loop}]"
    if isinstance(value, Carried):
        return f"carried[{value.loop},{value.slot}]"
    if isinstance(value, (tuple, list)):
        return "(" + ",".join(map(_digest_of, value)) + ")"
    if isinstance(value, slice):
        return f"slice[{_digest_of(value.start)}:{_digest_of(value.stop)}:{_digest_of(value.step)}]"
    if isinstance(value, float):
        return f"f{value!r}"
    if isinstance(value, (bool, int, str, type(None))):
        return f"{type(value).__name__}:{value!r}"
    raise TracingError(f"Value of type `{type(value).__name__}` cannot appear in a program.")


def _short(value):
    if isinstance(value, Node):
        return f"{value.op}#{value.digest[:6]}"
    try:
        return _digest_of(value)
    except TracingError:
        return repr(value)


class Program:
    """The traced application."""

    def __init__(self, params, stores):
        self.params = params  # list of ("tensor" | "scalar", constexpr flag)
        self.stores = stores  # list of (TensorRef, value)

    @property
    def digest(self):
        parts = [f"{kind}:{int(bool(constexpr))}" for kind, constexpr in self.params]
        for ref, value in self.stores:
            parts.append("store(" + _digest_of(ref) + "," + _digest_of(value) + ")")
        return hashlib.sha1("|".join(parts).encode()).hexdigest()[:20]

    def describe(self):
        """A readable dump of the graph (one line per node, stores last)."""
        lines, seen = [], set()

        def visit(value):
            if isinstance(value, (tuple, list)):
                for item in value:
                    visit(item)
            elif isinstance(value, TensorRef):
                visit(value.indices)
            elif isinstance(value, Node) and value.digest not in seen:
                seen.add(value.digest)
                for arg in value.args:
                    visit(arg)
                lines.append(f"{value.digest[:6]} = {value!r}")

        for ref, value in self.stores:
            visit(value)
            lines.append(f"store {_short(ref)} <- {_short(value)}")
        return "\n".join(lines)


# ---- the interpreter --------------------------------------------------------

_BINOPS = {
    ast.Add: ("add", lambda a, b: a + b),
    ast.Sub: ("sub", lambda a, b: a - b),
    ast.Mult: ("mul", lambda a, b: a * b),
    ast.Div: ("div", lambda a, b: a / b),
    ast.FloorDiv: ("floordiv", lambda a, b: a // b),
    ast.Mod: ("mod", lambda a, b: a % b),
    ast.Pow: ("pow", lambda a, b: a**b),
    ast.BitAnd: ("and", lambda a, b: a & b),
    ast.BitOr: ("or", lambda a, b: a | b),
    ast.LShift: ("shl", lambda a, b: a << b),
    ast.RShift: ("shr", lambda a, b: a >> b),
}

_COMPARES = {
    ast.Lt: ("lt", lambda a, b: a < b),
    ast.LtE: ("le", lambda a, b: a <= b),
    ast.Gt: ("gt", lambda a, b: a > b),
    ast.GtE: ("ge", lambda a, b: a >= b),
    ast.Eq: ("eq", lambda a, b: a == b),
    ast.NotEq: ("ne", lambda a, b: a != b),
}

_UNARY = {
    ast.USub: ("neg", lambda a: -a),
    ast.UAdd: ("pos", lambda a: +a),
    ast.Not: ("not", lambda a: not a),
    ast.Invert: ("invert", lambda a: ~a),
}

_PYTHON_CONSTANTS = (bool, int, float, str, type(None))


def _is_constant(value):
    if isinstance(value, _PYTHON_CONSTANTS):
        return True
    if isinstance(value, (tuple, list)):
        return all(_is_constant(item) for item in value)
    return False


class _Frame:
    def __init__(self, func, parent=None):
        self.func = func
        self.locals = {}
        self.aliases = {}  # parameter name -> (caller frame, caller name)
        self.parent = parent
        self.returned = None

    def lookup(self, name):
        if name in self.locals:
            return self.locals[name]
        func = self.func
        if func.__closure__:
            for cell_name, cell in zip(func.__code__.co_freevars, func.__closure__):
                if cell_name == name:
                    return cell.cell_contents
        if name in func.__globals__:
            return func.__globals__[name]
        if hasattr(builtins, name):
            return getattr(builtins, name)
        raise TracingError(f"Name `{name}` is not defined in the application.")


class Tracer:
    """Traces ``func`` whose parameters are bound to ``types`` (arranged
    tensors for tensor parameters, zero-dimensional tensors for scalars)."""

    def __init__(self, func, types):
        self.func = func
        self.types = list(types)
        self.stores = []
        self.num_loops = 0

    def run(self):
        parameters = list(inspect.signature(self.func).parameters)
        if len(parameters) != len(self.types):
            raise TracingError(
                f"The application takes {len(parameters)} parameters but the arrangement produced {len(self.types)} tensors."
            )
        frame = _Frame(self.func)
        self.param_values = {}
        kinds = []
        for position, (name, tensor) in enumerate(zip(parameters, self.types)):
            if not isinstance(tensor, Tensor):
                raise TracingError(f"Parameter `{name}` is not bound to a tensor.")
            if tensor.ndim == 0 and not isinstance(tensor.dtype, Tensor):
                value = ScalarParam(position, bool(tensor.constexpr))
                kinds.append(("scalar", tensor.constexpr))
            else:
                # an untiled tensor is a grid of single elements (every program gets a scalar)
                value = TensorRef(position, tensor.dtype if isinstance(tensor.dtype, Tensor) else _ELEMENT, 1)
                kinds.append(("tensor", False))
            frame.locals[name] = value
            self.param_values[name] = value
        self.top = frame
        self._exec_body(_function_tree(self.func).body, frame)
        return Program(kinds, self.stores)

    # ---- statements ------------------------------------------------------
    def _exec_body(self, body, frame):
        for statement in body:
            if frame.returned is not None:
                break
            self._exec(statement, frame)

    def _exec(self, node, frame):
        if isinstance(node, ast.Assign):
            value = self._eval(node.value, frame)
            for target in node.targets:
                self._assign(target, value, frame)
        elif isinstance(node, ast.AnnAssign):
            if node.value is not None:
                self._assign(node.target, self._eval(node.value, frame), frame)
        elif isinstance(node, ast.AugAssign):
            current = self._eval(_as_load(node.target), frame)
            value = self._binary(type(node.op), current, self._eval(node.value, frame))
            self._assign(node.target, value, frame)
        elif isinstance(node, ast.For):
            self._exec_for(node, frame)
        elif isinstance(node, ast.If):
            self._exec_if(node, frame)
        elif isinstance(node, ast.Expr):
            if not (isinstance(node.value, ast.Constant) and isinstance(node.value.value, str)):
                self._eval(node.value, frame)
        elif isinstance(node, ast.Return):
            frame.returned = (self._eval(node.value, frame) if node.value is not None else None,)
        elif isinstance(node, ast.Pass):
            pass
        else:
            raise TracingError(f"Statement `{type(node).__name__}` is not supported in an application.")

    def _assign(self, target, value, frame):
        if isinstance(target, ast.Name):
            self._assign_name(target.id, value, frame)
        elif isinstance(target, (ast.Tuple, ast.List)):
            if not isinstance(value, (tuple, list)) or len(value) != len(target.elts):
                raise TracingError("Cannot unpack a traced value.")
            for element, item in zip(target.elts, value):
                self._assign(element, item, frame)
        elif isinstance(target, ast.Subscript):
            ref = self._eval(_as_load(target), frame)
            if isinstance(ref, Node) and ref.op == "source_at":
                self.stores.append((ref, self._value(value)))
                return
            if not isinstance(ref, TensorRef) or not ref.is_tile:
                raise TracingError("Only tiles of tensor parameters can be assigned through a subscript.")
            self.stores.append((ref, self._value(value)))
        else:
            raise TracingError(f"Cannot assign to `{type(target).__name__}`.")

    def _assign_name(self, name, value, frame):
        if name in frame.aliases:  # a helper assigning to its parameter rebinds the caller's variable
            caller, caller_name = frame.aliases[name]
            frame.locals[name] = value
            self._assign_name(caller_name, value, caller)
            return
        if frame is self.top and name in self.param_values and isinstance(self.param_values[name], TensorRef):
            ref = self.param_values[name]
            if not ref.is_tile:
                raise TracingError(f"`{name}` is not a tile; index it before assigning.")
            self.stores.append((ref, self._value(value)))
            return
        frame.locals[name] = value

    def _exec_for(self, node, frame):
        if node.orelse:
            raise TracingError("`for ... else` is not supported.")
        iterable = self._eval(node.iter, frame)
        if not isinstance(iterable, _Range):
            raise TracingError("Loops must iterate over `range(...)`.")
        if not isinstance(node.target, ast.Name):
            raise TracingError("The loop variable must be a plain name.")
        if _is_constant(iterable.extent):  # a Python-level loop: unroll
            for i in range(iterable.extent):
                frame.locals[node.target.id] = i
                self._exec_body(node.body, frame)
            return

        loop = self.num_loops
        self.num_loops += 1
        carried = []
        for name in _assigned_names(node.body):
            if name in frame.locals and name not in carried and name != node.target.id:
                if isinstance(frame.locals[name], TensorRef):
                    continue  # assignments to tensor parameters are stores
                carried.append(name)
        # slots are numbered by what the names hold on entry (ties: first assignment in the body), so that
        # two bodies with the same dataflow get the same graph whatever the order of their statements
        carried.sort(key=lambda name: _digest_of(self._value(frame.locals[name])))
        initial = [frame.locals[name] for name in carried]
        for slot, name in enumerate(carried):
            frame.locals[name] = Carried(loop, slot)
        frame.locals[node.target.id] = LoopVar(loop)
        num_stores = len(self.stores)
        self._exec_body(node.body, frame)
        body_stores = self.stores[num_stores:]
        del self.stores[num_stores:]
        updates = [frame.locals[name] for name in carried]
        loop_node = Node(
            "loop",
            iterable.extent,
            tuple(self._value(v) for v in initial),
            tuple(self._value(v) for v in updates),
            tuple((ref, value) for ref, value in body_stores),
        )
        for slot, name in enumerate(carried):
            frame.locals[name] = Node("loop_out", loop_node, slot)
        if body_stores:
            self.stores.append((TensorRef(-1, Tensor(0), 0), loop_node))

    def _exec_if(self, node, frame):
        condition = self._eval(node.test, frame)
        if _is_constant(condition):
            self._exec_body(node.body if condition else node.orelse, frame)
            return
        condition = self._value(condition)
        before = dict(frame.locals)
        num_stores = len(self.stores)
        self._exec_body(node.body, frame)
        then_locals = frame.locals
        frame.locals = dict(before)
        self._exec_body(node.orelse, frame)
        else_locals = frame.locals
        if len(self.stores) != num_stores:
            raise TracingError("Stores inside a data-dependent `if` are not supported.")
        merged = dict(before)
        for name in set(then_locals) | set(else_locals):
            a = then_locals.get(name, before.get(name))
            b = else_locals.get(name, before.get(name))
            if a is b:
                merged[name] = a
            elif a is None or b is None:
                continue  # defined in one branch only: not visible afterwards
            else:
                merged[name] = Node("select", condition, self._value(a), self._value(b))
        frame.locals = merged

    # ---- expressions -------------------------------------------------------
    def _value(self, value):
        """Turns a tile reference used as a value into a load."""
        if isinstance(value, TensorRef):
            if not value.is_tile:
                raise TracingError("A tensor level was used as a value before being indexed down to a tile.")
            return Node("load", value)
        if isinstance(value, (tuple, list)):
            return tuple(self._value(item) for item in value)
        return value

    def _binary(self, op_type, lhs, rhs):
        name, function = _BINOPS[op_type]
        if _is_constant(lhs) and _is_constant(rhs):
            return function(lhs, rhs)
        return Node(name, self._value(lhs), self._value(rhs))

    def _eval(self, node, frame):
        method = getattr(self, "_eval_" + type(node).__name__, None)
        if method is None:
            raise TracingError(f"Expression `{type(node).__name__}` is not supported in an application.")
        return method(node, frame)

    def _eval_Constant(self, node, frame):
        return node.value

    def _eval_Name(self, node, frame):
        return frame.lookup(node.id)

    def _eval_Tuple(self, node, frame):
        return tuple(self._eval(element, frame) for element in node.elts)

    _eval_List = _eval_Tuple

    def _eval_Slice(self, node, frame):
        parts = [self._eval(part, frame) if part is not None else None for part in (node.lower, node.upper, node.step)]
        return slice(*parts)

    def _eval_BinOp(self, node, frame):
        return self._binary(type(node.op), self._eval(node.left, frame), self._eval(node.right, frame))

    def _eval_UnaryOp(self, node, frame):
        name, function = _UNARY[type(node.op)]
        operand = self._eval(node.operand, frame)
        if _is_constant(operand):
            return function(operand)
        return Node(name, self._value(operand))

    def _eval_Compare(self, node, frame):
        if len(node.ops) != 1:
            raise TracingError("Chained comparisons are not supported.")
        name, function = _COMPARES[type(node.ops[0])]
        lhs = self._eval(node.left, frame)
        rhs = self._eval(node.comparators[0], frame)
        if _is_constant(lhs) and _is_constant(rhs):
            return function(lhs, rhs)
        return Node(name, self._value(lhs), self._value(rhs))

    def _eval_BoolOp(self, node, frame):
        values = [self._eval(value, frame) for value in node.values]
        if all(_is_constant(value) for value in values):
            result = values[0]
            for value in values[1:]:
                result = (result and value) if isinstance(node.op, ast.And) else (result or value)
            return result
        name = "and" if isinstance(node.op, ast.And) else "or"
        result = self._value(values[0])
        for value in values[1:]:
            result = Node(name, result, self._value(value))
        return result

    def _eval_IfExp(self, node, frame):
        condition = self._eval(node.test, frame)
        if _is_constant(condition):
            return self._eval(node.body if condition else node.orelse, frame)
        return Node("select", self._value(condition), self._value(self._eval(node.body, frame)), self._value(self._eval(node.orelse, frame)))

    def _eval_Attribute(self, node, frame):
        base = self._eval(node.value, frame)
        attr = node.attr
        if isinstance(base, TensorRef):
            if attr == "shape":
                return tuple(Dim(base.param, base.level, d) for d in range(base.tensor.ndim))
            if attr == "ndim":
                return base.tensor.ndim
            if attr == "dtype":
                if base.is_tile:
                    return ElementType(base.param)
                raise TracingError("`.dtype` of a level that is not a tile; index it instead.")
            if attr == "source":
                return SourceRef(base.param)
            if attr in ("to", "offsets", "data_ptr", "stride"):
                return _BoundMethod(base, attr)
            raise TracingError(f"Tensors have no attribute `{attr}` in an application.")
        if isinstance(base, SourceRef):
            if attr == "shape":
                return _SourceShape(base.param, self.types[base.param].source.ndim)
            if attr == "ndim":
                return self.types[base.param].source.ndim
            if attr in ("data_ptr", "stride"):
                return _BoundMethod(base, attr)
            raise TracingError(f"`.source` has no attribute `{attr}`.")
        if isinstance(base, Node):
            if attr == "to":
                return _BoundMethod(base, attr)
            if attr == "shape" and base.op in ("zeros", "full"):
                return base.args[0]
            if attr == "dtype":
                return Node("dtype_of", base)
            raise TracingError(f"Traced values have no attribute `{attr}`.")
        if isinstance(base, ScalarParam) and attr == "to":
            return _BoundMethod(base, attr)
        try:
            return getattr(base, attr)
        except AttributeError:
            raise TracingError(f"`{base!r}` has no attribute `{attr}`.") from None

    def _eval_Subscript(self, node, frame):
        base = self._eval(node.value, frame)
        key = self._eval(node.slice, frame)
        if isinstance(base, TensorRef):
            keys = key if isinstance(key, tuple) else (key,)
            if base.is_tile:
                return Node("index", Node("load", base), tuple(keys))
            if len(keys) != base.tensor.ndim:
                raise TracingError(f"A level with {base.tensor.ndim} dimensions needs {base.tensor.ndim} indices, got {len(keys)}.")
            return TensorRef(base.param, base.tensor.dtype, base.level + 1, base.indices + tuple(self._value(k) for k in keys))
        if isinstance(base, SourceRef):  # `x.source[rows, columns]`: elements of the whole tensor by index
            return Node("source_at", base, self._source_indices(base, key))
        if isinstance(base, _SourceShape):
            if not isinstance(key, int):
                raise TracingError("Source shapes are indexed with integer constants.")
            return SourceDim(base.param, key % base.ndim)
        if isinstance(base, Node):
            keys = key if isinstance(key, tuple) else (key,)
            return Node("index", base, tuple(keys))
        if isinstance(base, (tuple, list)) and _is_constant(key):
            return base[key]
        if _is_constant(base) and _is_constant(key):
            return base[key]
        raise TracingError("Unsupported subscript in an application.")

    def _source_indices(self, source, key):
        keys = key if isinstance(key, tuple) else (key,)
        ndim = self.types[source.param].source.ndim
        if len(keys) != ndim:
            raise TracingError(f"A source tensor with {ndim} dimensions needs {ndim} indices, got {len(keys)}.")
        return tuple(self._value(k) for k in keys)

    def _eval_Call(self, node, frame):
        func = self._eval(node.func, frame)
        args = [self._eval(arg, frame) for arg in node.args]
        kwargs = {keyword.arg: self._eval(keyword.value, frame) for keyword in node.keywords}
        if any(keyword.arg is None for keyword in node.keywords):
            raise TracingError("`**kwargs` is not supported in an application.")

        if language.is_function(func) and func.name in ("store", "atomic_add"):
            # `ntl.store(pointer, value)` / `ntl.atomic_add(pointer, value)`: a store through a raw pointer
            if len(args) != 2 or kwargs:
                raise TracingError(f"`ntl.{func.name}` takes a pointer and a value.")
            self.stores.append((Node("pointer_" + func.name, self._value(args[0])), self._value(args[1])))
            return None
        if language.is_function(func):
            # one spelling per call: trailing positional arguments that have a name become keywords,
            # `dot(a, b, acc)` is `acc + dot(a, b)` (so equivalent applications share a digest)
            args, kwargs = list(args), dict(kwargs)
            names = _TRAILING_PARAMETERS.get(func.name)
            if names is not None:
                first, trailing = names
                for name, value in zip(trailing, args[first:]):
                    if name in kwargs:
                        raise TracingError(f"`ntl.{func.name}` got `{name}` twice.")
                    kwargs[name] = value
                del args[first:]
            accumulator = kwargs.pop("acc", None) if func.name == "dot" else None
            items = tuple(self._value(arg) for arg in args)
            named = tuple(sorted((name, self._value(value)) for name, value in kwargs.items() if not (name == "keep_dims" and value is False) and not (name == "axis" and value is None)))
            node = Node(func.name, *items, *[Node("kwarg", name, value) for name, value in named])
            if accumulator is not None:
                node = Node("add", self._value(accumulator), node)
            return node
        if isinstance(func, _BoundMethod):
            return self._call_method(func, args, kwargs)
        if func is range:
            if len(args) != 1 or kwargs:
                raise TracingError("Only `range(stop)` is supported.")
            return _Range(args[0])
        if isinstance(func, types.FunctionType):
            return self._inline(func, node, args, kwargs, frame)
        if callable(func) and all(_is_constant(arg) for arg in args) and all(_is_constant(v) for v in kwargs.values()):
            return func(*args, **kwargs)
        raise TracingError(f"Cannot call `{func!r}` inside an application.")

    def _call_method(self, method, args, kwargs):
        base, name = method.base, method.name
        if name == "to":
            if len(args) != 1 or kwargs:
                raise TracingError("`.to` takes exactly one dtype.")
            return Node("cast", self._value(base), args[0])
        if name == "offsets":
            if not isinstance(base, TensorRef):
                raise TracingError("`.offsets` applies to tensor parameters.")
            dim = args[0] if args else kwargs.get("dim")
            source_ndim = self.types[base.param].source.ndim
            if dim is None:
                return Node("offsets", base, None)
            if not isinstance(dim, int):
                raise TracingError("`.offsets(dim)` needs an integer constant.")
            return Node("offsets", base, dim % source_ndim)
        if name == "data_ptr":
            if not isinstance(base, SourceRef) or args or kwargs:
                raise TracingError("`.data_ptr()` applies to `tensor.source`.")
            return Node("data_ptr", base)
        if name == "stride":
            if not isinstance(base, SourceRef) or len(args) != 1 or not isinstance(args[0], int):
                raise TracingError("`.source.stride(dim)` needs an integer constant.")
            return SourceStride(base.param, args[0] % self.types[base.param].source.ndim)
        raise TracingError(f"Method `{name}` is not supported in an application.")

    def _inline(self, func, call, args, kwargs, frame):
        signature = inspect.signature(func)
        try:
            bound = signature.bind(*args, **kwargs)
        except TypeError as error:
            raise TracingError(str(error)) from None
        bound.apply_defaults()
        callee = _Frame(func, parent=frame)
        callee.locals.update(bound.arguments)
        parameters = list(signature.parameters)
        for position, arg in enumerate(call.args):
            if isinstance(arg, ast.Name) and position < len(parameters):
                callee.aliases[parameters[position]] = (frame, arg.id)
        for keyword in call.keywords:
            if isinstance(keyword.value, ast.Name):
                callee.aliases[keyword.arg] = (frame, keyword.value.id)
        self._exec_body(_function_tree(func).body, callee)
        return callee.returned[0] if callee.returned is not None else None


# language functions whose trailing positional parameters have names: (leading positional count, names)
_TRAILING_PARAMETERS = {
    "zeros": (1, ("dtype",)),
    "full": (2, ("dtype",)),
    "sum": (1, ("axis", "keep_dims")),
    "max": (1, ("axis", "keep_dims")),
    "min": (1, ("axis", "keep_dims")),
    "dot": (2, ("acc",)),
}


class _BoundMethod:
    __slots__ = ("base", "name")

    def __init__(self, base, name):
        self.base, self.name = base, name


class _SourceShape:
    __slots__ = ("param", "ndim")

    def __init__(self, param, ndim):
        self.param, self.ndim = param, ndim


def _as_load(target):
    clone = ast.parse(ast.unparse(target), mode="eval").body
    return clone


def _assigned_names(body):
    names = []
    for statement in body:
        for node in ast.walk(statement):
            targets = []
            if isinstance(node, ast.Assign):
                targets = node.targets
            elif isinstance(node, (ast.AugAssign, ast.AnnAssign)):
                targets = [node.target]
            for target in targets:
                for leaf in ast.walk(target):
                    if isinstance(leaf, ast.Name) and isinstance(leaf.ctx, ast.Store) and leaf.id not in names:
                        names.append(leaf.id)
    return names


_TREE_CACHE = {}


def _function_tree(func):
    key = func.__code__
    if key not in _TREE_CACHE:
        try:
            source = textwrap.dedent(inspect.getsource(func))
        except (OSError, TypeError) as error:
            raise TracingError(f"The source of `{getattr(func, '__name__', func)}` is not available.") from error
        tree = ast.parse(source)
        definition = next((n for n in ast.walk(tree) if isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef))), None)
        if definition is None:
            raise TracingError("Applications must be defined with `def`.")
        _TREE_CACHE[key] = definition
    return _TREE_CACHE[key]


def trace(application, types):
    """Traces ``application`` with its parameters bound to ``types``."""
    return Tracer(application, types).run()
