"""Symbolic integers for arrangements.

A :class:`Symbol` is an immutable expression tree over named integers
(tensor sizes and strides, block sizes, call-time constants, tile index
variables).  Arrangements build such expressions while they run on symbolic
tensors; they are evaluated -- with plain ints or with numpy arrays -- once a
kernel is called with concrete tensors.

Mirrors the user-facing behaviour of the reference's ``Symbol`` and
``block_size`` (reference: src/ninetoothed/symbol.py:9-268): the constructor
flags ``constexpr`` / ``meta`` / ``lower_bound`` / ``upper_bound`` /
``power_of_two`` with the same defaults, operator overloads with the same
identity folding (``+ 0``, ``* 1``, ``// 1``), structural ``==`` that returns a
plain ``bool``.  The representation is a tuple tree rather than Python ``ast``
nodes, because nothing here is ever turned back into source code.
"""

import numbers
import operator

import numpy as np

_BINARY = {
    "+": operator.add,
    "-": operator.sub,
    "*": operator.mul,
    "//": operator.floordiv,
    "%": operator.mod,
    "<": operator.lt,
    "<=": operator.le,
    ">": operator.gt,
    ">=": operator.ge,
    "&": operator.and_,
    "|": operator.or_,
}

# defaults of the reference (src/ninetoothed/symbol.py:59-65)
_META_LOWER, _META_UPPER = 2**5, 2**10
_CONSTEXPR_LOWER, _CONSTEXPR_UPPER = 1, 2**20


class Symbol:
    """A symbolic integer (or boolean) expression.

    :param expr: A name, a number, or another :class:`Symbol`.
    :param constexpr: Whether the name is a call-time constant.
    :param meta: Whether the name is a tunable meta-parameter (block size).
    :param lower_bound: Smallest admissible value.
    :param upper_bound: Largest admissible value.
    :param power_of_two: Whether the value has to be a power of two.
    """

    __slots__ = ("_node", "constexpr", "meta", "lower_bound", "upper_bound", "power_of_two")

    def __init__(self, expr, constexpr=None, meta=None, lower_bound=None, upper_bound=None, power_of_two=None):
        self.constexpr = None
        self.meta = None
        self.lower_bound = None
        self.upper_bound = None
        self.power_of_two = None

        if isinstance(expr, Symbol):
            self._node = expr._node
            for slot in ("constexpr", "meta", "lower_bound", "upper_bound", "power_of_two"):
                setattr(self, slot, getattr(expr, slot))
            return

        if isinstance(expr, tuple):  # internal: already a node
            self._node = expr
            return

        if isinstance(expr, (bool, np.bool_)):
            self._node = ("const", bool(expr))
        elif isinstance(expr, numbers.Integral):
            self._node = ("const", int(expr))
        elif isinstance(expr, numbers.Real):
            self._node = ("const", float(expr))
        elif isinstance(expr, str):
            text = expr.strip()
            try:
                self._node = ("const", int(text))
            except ValueError:
                if not text.isidentifier():
                    raise ValueError(f"`{expr}` is not a valid symbol name.")
                self._node = ("name", text, self)
        else:
            raise TypeError(f"Cannot make a symbol from `{type(expr).__name__}`.")

        if (constexpr or meta) and self._node[0] != "name":
            raise ValueError("`constexpr` and `meta` are properties of name symbols.")

        if meta and constexpr is False:
            raise ValueError("Non-constexpr meta symbol is not supported.")

        self.meta = bool(meta) if meta is not None else None
        self.constexpr = True if meta else constexpr

        if meta:
            defaults = (_META_LOWER, _META_UPPER, True)
        elif constexpr:
            defaults = (_CONSTEXPR_LOWER, _CONSTEXPR_UPPER, False)
        else:
            defaults = (None, None, None)

        self.lower_bound = lower_bound if lower_bound is not None else defaults[0]
        self.upper_bound = upper_bound if upper_bound is not None else defaults[1]
        self.power_of_two = power_of_two if power_of_two is not None else defaults[2]

    # ---- structure -------------------------------------------------------
    @property
    def kind(self):
        return self._node[0]

    @property
    def is_constant(self):
        return self._node[0] == "const"

    @property
    def is_name(self):
        return self._node[0] == "name"

    @property
    def value(self):
        if not self.is_constant:
            raise ValueError(f"`{self}` is not a constant.")
        return self._node[1]

    @property
    def name(self):
        if not self.is_name:
            raise ValueError(f"`{self}` is not a name.")
        return self._node[1]

    @property
    def op(self):
        return self._node[0]

    @property
    def operands(self):
        if self._node[0] in ("const", "name"):
            return ()
        return self._node[1:]

    def _key(self):
        node = self._node
        if node[0] == "const":
            return node
        if node[0] == "name":
            return ("name", node[1])
        return (node[0],) + tuple(child._key() for child in node[1:])

    def __eq__(self, other):
        if isinstance(other, Symbol):
            return self._key() == other._key()
        if isinstance(other, numbers.Number) and self.is_constant:
            return self._node[1] == other
        return False

    def __ne__(self, other):
        return not self.__eq__(other)

    def __hash__(self):
        return hash(self._key())

    def __bool__(self):
        if self.is_constant:
            return bool(self._node[1])
        raise TypeError(f"The truth value of the symbolic expression `{self}` is not known.")

    def __index__(self):
        if self.is_constant and isinstance(self._node[1], int):
            return self._node[1]
        raise TypeError(f"`{self}` is not a concrete integer.")

    __int__ = __index__

    # ---- construction ----------------------------------------------------
    @staticmethod
    def _wrap(value):
        return value if isinstance(value, Symbol) else Symbol(value)

    @staticmethod
    def _binary(op, lhs, rhs):
        lhs, rhs = Symbol._wrap(lhs), Symbol._wrap(rhs)
        if lhs.is_constant and rhs.is_constant:
            return Symbol(_BINARY[op](lhs.value, rhs.value))
        return Symbol((op, lhs, rhs))

    def __add__(self, other):
        other = Symbol._wrap(other)
        if self == 0:
            return other
        if other == 0:
            return self
        return Symbol._binary("+", self, other)

    def __radd__(self, other):
        return Symbol._wrap(other).__add__(self)

    def __sub__(self, other):
        other = Symbol._wrap(other)
        if other == 0:
            return self
        return Symbol._binary("-", self, other)

    def __rsub__(self, other):
        return Symbol._wrap(other).__sub__(self)

    def __neg__(self):
        return Symbol._binary("-", 0, self)

    def __mul__(self, other):
        other = Symbol._wrap(other)
        if self == 1:
            return other
        if other == 1:
            return self
        if self == 0 or other == 0:
            return Symbol(0)
        return Symbol._binary("*", self, other)

    def __rmul__(self, other):
        return Symbol._wrap(other).__mul__(self)

    def __floordiv__(self, other):
        other = Symbol._wrap(other)
        if other == 1:
            return self
        return Symbol._binary("//", self, other)

    def __rfloordiv__(self, other):
        return Symbol._wrap(other).__floordiv__(self)

    def __mod__(self, other):
        return Symbol._binary("%", self, other)

    def __rmod__(self, other):
        return Symbol._wrap(other).__mod__(self)

    def __lt__(self, other):
        return Symbol._binary("<", self, other)

    def __le__(self, other):
        return Symbol._binary("<=", self, other)

    def __gt__(self, other):
        return Symbol._binary(">", self, other)

    def __ge__(self, other):
        return Symbol._binary(">=", self, other)

    def __and__(self, other):
        return Symbol._binary("&", self, other)

    def __rand__(self, other):
        return Symbol._wrap(other).__and__(self)

    def __or__(self, other):
        return Symbol._binary("|", self, other)

    # ---- evaluation ------------------------------------------------------
    def names(self):
        """The set of name symbols this expression mentions."""
        found = {}
        stack = [self]
        while stack:
            current = stack.pop()
            if current.is_name:
                found.setdefault(current.name, current._node[2])
            else:
                stack.extend(current.operands)
        return set(found.values())

    def evaluate(self, env):
        """Evaluates with ``env`` mapping names to numbers or numpy arrays."""
        node = self._node
        if node[0] == "const":
            return node[1]
        if node[0] == "name":
            try:
                return env[node[1]]
            except KeyError:
                raise KeyError(f"No value given for symbol `{node[1]}`.") from None
        lhs = node[1].evaluate(env)
        rhs = node[2].evaluate(env)
        return _BINARY[node[0]](lhs, rhs)

    def substitute(self, mapping):
        """Replaces names by symbols / numbers; ``mapping`` is keyed by name."""
        node = self._node
        if node[0] == "const":
            return self
        if node[0] == "name":
            return Symbol._wrap(mapping[node[1]]) if node[1] in mapping else self
        lhs = node[1].substitute(mapping)
        rhs = node[2].substitute(mapping)
        method = {
            "+": Symbol.__add__,
            "-": Symbol.__sub__,
            "*": Symbol.__mul__,
            "//": Symbol.__floordiv__,
            "%": Symbol.__mod__,
        }.get(node[0])
        if method is not None:
            return method(lhs, rhs)
        return Symbol._binary(node[0], lhs, rhs)

    def __repr__(self):
        node = self._node
        if node[0] == "const":
            return repr(node[1])
        if node[0] == "name":
            return node[1]
        return f"({node[1]!r} {node[0]} {node[2]!r})"


def block_size(lower_bound=None, upper_bound=None):
    """Creates a tunable block-size symbol (a meta-parameter).

    Same contract as the reference's ``block_size``
    (src/ninetoothed/symbol.py:253-268): a fresh power-of-two meta symbol per
    call, by default in ``[32, 1024]``.
    """

    name = f"ninetoothed_BLOCK_SIZE_{block_size._num_block_sizes}"
    block_size._num_block_sizes += 1
    return Symbol(name, meta=True, lower_bound=lower_bound, upper_bound=upper_bound)


block_size._num_block_sizes = 0


def evaluate(value, env):
    """Evaluates a Symbol, or passes a plain number through."""
    if isinstance(value, Symbol):
        return value.evaluate(env)
    return value
