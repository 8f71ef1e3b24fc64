"""Integers that remember how they were computed from the sizes of a call.

A packaged element-wise kernel has to lower its program for sizes that are only known when the
C launch function runs, without Python.  The lowering (``ninetoothed_amd.mapping``) is ordinary
integer arithmetic on sizes and strides plus decisions taken by comparing them, so it is run
once on sample sizes with :class:`SymInt` values: every ``+ - * // %`` result carries its
expression in the call's sizes, and every decision (a comparison, a truth test, a use as an
index or a conversion) is recorded as a *guard* together with its outcome.  The program built
from the sample is then right for every call whose sizes give the same outcomes, with the
recorded expressions in place of the sample's numbers -- the packaged C code evaluates the
guards and the expressions (``ninetoothed_amd.aot``).

Nothing here is specific to that use: a :class:`SymInt` behaves like the ``int`` it holds.
One use escapes the record: CPython reads an ``int`` subclass directly when it serves as a
sequence index or in ``range()``, without calling a method, so code that is to be run on
symbolic sizes must not do that with them (the lowering only counts ranks and operands that way).
"""

import functools
import operator

_recorder = None


class Recorder:
    """Collects the guards of the arithmetic done while it is active (``with Recorder() as r``)."""

    def __init__(self):
        self.guards = {}  # (operator, lhs expression, rhs expression) -> outcome

    def __enter__(self):
        global _recorder
        self._previous, _recorder = _recorder, self
        return self

    def __exit__(self, *exc_info):
        global _recorder
        _recorder = self._previous
        return False

    def record(self, op, lhs, rhs, outcome):
        known = self.guards.setdefault((op, lhs, rhs), outcome)
        assert known == outcome, "a comparison of the same expressions changed its outcome"


def plain(value):
    """The ``int`` a value holds, without recording anything."""
    return int.__add__(value, 0) if isinstance(value, int) else value


def is_symbolic(*values):
    return any(isinstance(value, SymInt) for value in values)


def expression(value):
    return value.expr if isinstance(value, SymInt) else ("const", plain(value))


def integer(value):
    """``int(value)`` that keeps a :class:`SymInt` as it is."""
    return value if isinstance(value, SymInt) else int(value)


def same(a, b):
    """Equality that decides nothing about a call: symbolic values are equal only when they
    are the same expression (so that values which merely coincide in the sample stay apart)."""
    if is_symbolic(a, b):
        return expression(a) == expression(b)
    return a == b


def same_structure(a, b):
    """:func:`same` over nested tuples (the keys of index expressions)."""
    if isinstance(a, tuple) and isinstance(b, tuple):
        return len(a) == len(b) and all(same_structure(x, y) for x, y in zip(a, b))
    if isinstance(a, tuple) or isinstance(b, tuple):
        return False
    if isinstance(a, int) and isinstance(b, int):
        return same(a, b)
    return a == b


@functools.lru_cache(maxsize=None)
def _linear(expr):
    """``expr`` as ``(constant, ((atom, coefficient), ...))``: sums, differences and products with
    a constant are expanded, everything else is an atom."""
    kind = expr[0]
    if kind == "const":
        return expr[1], ()
    if kind in ("+", "-", "*"):
        (c1, t1), (c2, t2) = _linear(expr[1]), _linear(expr[2])
        if kind == "*":
            if t1 and t2:
                return 0, ((expr, 1),)
            factor, (constant, terms) = (c1, (c2, t2)) if not t1 else (c2, (c1, t1))
            return constant * factor, tuple((atom, coef * factor) for atom, coef in terms if coef * factor)
        sign = 1 if kind == "+" else -1
        terms = dict(t1)
        for atom, coef in t2:
            terms[atom] = terms.get(atom, 0) + sign * coef
        return c1 + sign * c2, tuple((atom, coef) for atom, coef in terms.items() if coef)
    return 0, ((expr, 1),)


def constant_difference(a, b):
    """``a - b`` when that is the same number for every call, else ``None``."""
    constant, terms = _linear(("-", expression(a), expression(b)))
    return constant if not terms else None


def _guard(op, lhs, rhs, outcome):
    if not is_symbolic(lhs, rhs):
        return
    left, right = expression(lhs), expression(rhs)
    if left == right:
        return
    if _recorder is not None:
        _recorder.record(op, left, right, bool(outcome))


def _arithmetic(op, function, reflected=False):
    def method(self, other):
        if isinstance(other, float):
            return function(float(self), other) if not reflected else function(other, float(self))
        if not isinstance(other, int):
            return NotImplemented
        lhs, rhs = (other, self) if reflected else (self, other)
        if op in ("//", "%"):
            _guard("!=", rhs, 0, True)  # the packaged code must not divide by zero either
        value = function(plain(lhs), plain(rhs))
        if not isinstance(rhs, SymInt):
            constant = plain(rhs)
            if (op in ("+", "-") and constant == 0) or (op in ("*", "//") and constant == 1):
                return lhs
            if op == "*" and constant == 0:
                return 0
            if op == "%" and constant == 1:
                return 0
        elif not isinstance(lhs, SymInt):
            constant = plain(lhs)
            if (op == "+" and constant == 0) or (op == "*" and constant == 1):
                return rhs
            if op in ("*", "//", "%") and constant == 0:
                return 0
        left, right = expression(lhs), expression(rhs)
        if op in ("+", "-") and right[0] == "const":  # x + c, with the constants of nested sums folded
            constant = right[1] if op == "+" else -right[1]
            if left[0] == "+" and left[2][0] == "const":
                left, constant = left[1], left[2][1] + constant
            return SymInt(value, ("+", left, ("const", constant)) if constant else left)
        return SymInt(value, (op, left, right))

    return method


def _comparison(op, function):
    def method(self, other):
        if isinstance(other, float):
            return function(float(self), other)
        if not isinstance(other, int):
            return NotImplemented
        outcome = function(plain(self), plain(other))
        _guard(op, self, other, outcome)
        return outcome

    return method


def _specialising(name):
    """Operations without a symbolic form pin the value (guard: it equals the sample's)."""

    def method(self, *args):
        return getattr(int, name)(self.pin(), *(arg.pin() if isinstance(arg, SymInt) else arg for arg in args))

    return method


class SymInt(int):
    """An ``int`` with the expression it came from.  ``expr`` is a nested tuple:
    ``("sym", c_expression)``, ``("const", n)`` or ``(operator, lhs, rhs)``."""

    def __new__(cls, value, expr):
        self = super().__new__(cls, plain(value))
        self.expr = expr
        return self

    @staticmethod
    def symbol(c_expression, sample):
        return SymInt(sample, ("sym", c_expression))

    def pin(self):
        value = plain(self)
        _guard("==", self, value, True)
        return value

    __add__ = _arithmetic("+", operator.add)
    __radd__ = _arithmetic("+", operator.add, reflected=True)
    __sub__ = _arithmetic("-", operator.sub)
    __rsub__ = _arithmetic("-", operator.sub, reflected=True)
    __mul__ = _arithmetic("*", operator.mul)
    __rmul__ = _arithmetic("*", operator.mul, reflected=True)
    __floordiv__ = _arithmetic("//", operator.floordiv)
    __rfloordiv__ = _arithmetic("//", operator.floordiv, reflected=True)
    __mod__ = _arithmetic("%", operator.mod)
    __rmod__ = _arithmetic("%", operator.mod, reflected=True)

    def __neg__(self):
        return 0 - self

    def __pos__(self):
        return self

    def __abs__(self):
        return self if self >= 0 else -self

    __lt__ = _comparison("<", operator.lt)
    __le__ = _comparison("<=", operator.le)
    __gt__ = _comparison(">", operator.gt)
    __ge__ = _comparison(">=", operator.ge)
    __eq__ = _comparison("==", operator.eq)
    __ne__ = _comparison("!=", operator.ne)

    def __hash__(self):
        return hash(plain(self))

    def __bool__(self):
        return self != 0

    def __index__(self):
        return self.pin()

    def __int__(self):
        return self.pin()

    def __float__(self):
        return float(self.pin())

    def __repr__(self):
        return int.__repr__(self)

    __str__ = __repr__

    def __format__(self, spec):
        return format(plain(self), spec)

    def __reduce__(self):
        return (SymInt, (plain(self), self.expr))


for _name in (
    "__truediv__", "__rtruediv__", "__pow__", "__rpow__", "__divmod__", "__rdivmod__", "__lshift__", "__rlshift__", "__rshift__",
    "__rrshift__", "__and__", "__rand__", "__or__", "__ror__", "__xor__", "__rxor__", "__invert__", "__round__", "__trunc__",
    "__floor__", "__ceil__", "bit_length", "bit_count", "to_bytes", "conjugate",
):
    setattr(SymInt, _name, _specialising(_name))


# ---- C code for expressions and guards -----------------------------------------------------

C_HELPERS = (
    "static inline int64_t nt_floordiv(int64_t a, int64_t b) { int64_t q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }\n"
    "static inline int64_t nt_mod(int64_t a, int64_t b) { int64_t r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r; }\n"
)


class CWriter:
    """Turns expressions into C statements, one ``const int64_t`` per distinct sub-expression."""

    def __init__(self, prefix="t"):
        self.prefix = prefix
        self.names = {}
        self.lines = []

    def value(self, expr):
        kind = expr[0]
        if kind == "const":
            number = expr[1]
            if number == -(2**63):
                return "(-9223372036854775807LL - 1)"
            return f"INT64_C({number})" if number >= 0 else f"(-INT64_C({-number}))"
        if expr in self.names:
            return self.names[expr]
        if kind == "sym":
            text = f"(int64_t)({expr[1]})"
        else:
            lhs, rhs = self.value(expr[1]), self.value(expr[2])
            if kind == "+" and expr[2][0] == "const" and expr[2][1] < 0:
                kind, rhs = "-", self.value(("const", -expr[2][1]))
            if kind == "//":
                text = f"nt_floordiv({lhs}, {rhs})"
            elif kind == "%":
                text = f"nt_mod({lhs}, {rhs})"
            else:
                text = f"{lhs} {kind} {rhs}"
        name = f"{self.prefix}{len(self.names)}"
        self.names[expr] = name
        self.lines.append(f"const int64_t {name} = {text};")
        return name

    def failure(self, key, outcome):
        """Emits the sub-expressions of a guard and returns the C condition under which it does
        *not* hold.  Guards are emitted in the order they were recorded, one ``if`` each, so the
        statements of a division run only after the check of its divisor."""
        op, lhs, rhs = key
        text = f"{self.value(lhs)} {op} {self.value(rhs)}"
        return f"!({text})" if outcome else text

    def take_lines(self):
        lines, self.lines = self.lines, []
        return lines


def evaluate(expr, symbols):
    """Value of an expression for ``symbols`` (C expression text -> int); the check the
    packaging tests use against a second lowering."""
    kind = expr[0]
    if kind == "const":
        return expr[1]
    if kind == "sym":
        return symbols[expr[1]]
    lhs, rhs = evaluate(expr[1], symbols), evaluate(expr[2], symbols)
    return {"+": operator.add, "-": operator.sub, "*": operator.mul, "//": operator.floordiv, "%": operator.mod}[kind](lhs, rhs)


def holds(key, outcome, symbols):
    op, lhs, rhs = key
    compare = {"<": operator.lt, "<=": operator.le, ">": operator.gt, ">=": operator.ge, "==": operator.eq, "!=": operator.ne}[op]
    return compare(evaluate(lhs, symbols), evaluate(rhs, symbols)) == outcome
