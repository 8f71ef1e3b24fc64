"""Normal form for the index arithmetic arrangements produce.

Once the sizes of a call are known, every source index of an arranged tensor is
an integer expression in a handful of index variables built from ``+ - *``
with constants and ``//``, ``%`` by constants (``flatten`` decodes with div /
mod, everything else is linear; reference: src/ninetoothed/tensor.py:258-274,
462-471, 555-556, 712-716).  :class:`Affine` keeps such an expression as

    constant + sum(coefficient * atom)

where an atom is an index variable, ``floor(inner / c)`` or ``inner mod c``
with ``inner`` again an :class:`Affine`.  Division and modulo simplify with the
known ranges of the variables, so equal index maps get equal normal forms and
can be compared or pattern-matched structurally.
"""

from ninetoothed_amd.symbol import Symbol
from ninetoothed_amd.symbolic_int import integer, is_symbolic


class Affine:
    __slots__ = ("const", "terms")

    def __init__(self, const=0, terms=None):
        self.const = integer(const)
        self.terms = {atom: coef for atom, coef in (terms or {}).items() if coef != 0}

    # atoms: ("var", name) | ("div", key, c) | ("mod", key, c); `key` = Affine.key()
    def key(self):
        return (self.const, tuple(sorted(self.terms.items(), key=repr)))

    @staticmethod
    def from_key(key):
        return Affine(key[0], dict(key[1]))

    @staticmethod
    def var(name):
        return Affine(0, {("var", name): 1})

    def is_const(self):
        return not self.terms

    def coef(self, name):
        return self.terms.get(("var", name), 0)

    def __eq__(self, other):
        return isinstance(other, Affine) and self.key() == other.key()

    def __hash__(self):
        return hash(self.key())

    def __add__(self, other):
        other = _wrap(other)
        terms = dict(self.terms)
        for atom, coef in other.terms.items():
            terms[atom] = terms.get(atom, 0) + coef
        return Affine(self.const + other.const, terms)

    __radd__ = __add__

    def __neg__(self):
        return self * -1

    def __sub__(self, other):
        return self + (-_wrap(other))

    def __rsub__(self, other):
        return _wrap(other) - self

    def __mul__(self, factor):
        if isinstance(factor, Affine):
            if factor.is_const():
                factor = factor.const
            elif self.is_const():
                return factor * self.const
            else:
                raise NotAffine("product of two index expressions")
        return Affine(self.const * factor, {atom: coef * factor for atom, coef in self.terms.items()})

    __rmul__ = __mul__

    def variables(self):
        names = set()
        for atom in self.terms:
            if atom[0] == "var":
                names.add(atom[1])
            else:
                names |= Affine.from_key(atom[1]).variables()
        return names

    def is_linear(self):
        return all(atom[0] == "var" for atom in self.terms)

    def __repr__(self):
        parts = [str(self.const)] if self.const or not self.terms else []
        for atom, coef in sorted(self.terms.items(), key=repr):
            parts.append((f"{coef}*" if coef != 1 else "") + _atom_repr(atom))
        return " + ".join(parts)


def _atom_repr(atom):
    if atom[0] == "var":
        return atom[1]
    symbol = "//" if atom[0] == "div" else "%"
    return f"(({Affine.from_key(atom[1])!r}) {symbol} {atom[2]})"


class NotAffine(Exception):
    """The expression leaves the div/mod-affine class."""


def _wrap(value):
    return value if isinstance(value, Affine) else Affine(value)


def _split(expr, c):
    """``expr == c * quotient + remainder`` with every coefficient of
    ``remainder`` not divisible by ``c`` and its constant in ``[0, c)``."""
    quotient_terms, remainder_terms = {}, {}
    for atom, coef in expr.terms.items():
        # sizes only known at launch: any term may stay in the remainder, so nothing is decided from the sample
        if not is_symbolic(coef, c) and coef % c == 0:
            quotient_terms[atom] = coef // c
        else:
            remainder_terms[atom] = coef
    return Affine(expr.const // c, quotient_terms), Affine(expr.const % c, remainder_terms)


class Ranges:
    """Inclusive value ranges of index variables, and arithmetic under them."""

    def __init__(self, extents=None):
        self.bounds = {}
        for name, extent in (extents or {}).items():
            self.bounds[name] = (0, extent - 1)

    def copy(self):
        other = Ranges()
        other.bounds = dict(self.bounds)
        return other

    def interval(self, expr):
        expr = _wrap(expr)
        lo = hi = expr.const
        for atom, coef in expr.terms.items():
            a_lo, a_hi = self._atom_interval(atom)
            if coef >= 0:
                lo += coef * a_lo
                hi += coef * a_hi
            else:
                lo += coef * a_hi
                hi += coef * a_lo
        return lo, hi

    def _atom_interval(self, atom):
        if atom[0] == "var":
            return self.bounds[atom[1]]
        lo, hi = self.interval(Affine.from_key(atom[1]))
        c = atom[2]
        if atom[0] == "div":
            return lo // c, hi // c
        if lo // c == hi // c:
            return lo % c, hi % c
        return 0, c - 1

    def floordiv(self, expr, c):
        expr = _wrap(expr)
        if c <= 0:
            raise NotAffine("division by a non-positive constant")
        if not is_symbolic(c) and c == 1:
            return expr
        quotient, remainder = _split(expr, c)
        if remainder.is_const():
            return quotient + remainder.const // c
        lo, hi = self.interval(remainder)
        if not is_symbolic(lo, hi, c) and lo // c == hi // c:
            return quotient + lo // c
        if len(remainder.terms) == 1 and remainder.const == 0:
            (atom, coef), = remainder.terms.items()
            if coef == 1 and atom[0] == "div":  # (x // a) // c == x // (a * c)
                return quotient + self.floordiv(Affine.from_key(atom[1]), atom[2] * c)
        return quotient + Affine(0, {("div", remainder.key(), c): 1})

    def mod(self, expr, c):
        expr = _wrap(expr)
        if c <= 0:
            raise NotAffine("modulo by a non-positive constant")
        if not is_symbolic(c) and c == 1:
            return Affine(0)
        _, remainder = _split(expr, c)
        if remainder.is_const():
            return Affine(remainder.const % c)
        lo, hi = self.interval(remainder)
        if not is_symbolic(lo, hi, c) and lo // c == hi // c:
            return remainder - (lo // c) * c
        if len(remainder.terms) == 1 and remainder.const == 0:
            (atom, coef), = remainder.terms.items()
            if coef == 1 and atom[0] == "mod" and not is_symbolic(atom[2], c) and atom[2] % c == 0:  # (x % a) % c == x % c when c | a
                return self.mod(Affine.from_key(atom[1]), c)
        return Affine(0, {("mod", remainder.key(), c): 1})

    def convert(self, expr, env):
        """Normal form of a :class:`Symbol` expression.

        Names found in ``env`` are constants; all other names must be index
        variables with a known range.  A variable whose range is a single
        value is replaced by that value."""

        if not isinstance(expr, Symbol):
            return Affine(int(expr))
        if expr.is_constant:
            return Affine(int(expr.value))
        if expr.is_name:
            name = expr.name
            if name in env:
                return Affine(integer(env[name]))
            if name not in self.bounds:
                raise NotAffine(f"unknown symbol `{name}`")
            lo, hi = self.bounds[name]
            return Affine(lo) if not is_symbolic(lo, hi) and lo == hi else Affine.var(name)
        op = expr.op
        lhs = self.convert(expr.operands[0], env)
        rhs = self.convert(expr.operands[1], env)
        if op == "+":
            return lhs + rhs
        if op == "-":
            return lhs - rhs
        if op == "*":
            return lhs * rhs
        if op in ("//", "%"):
            if not rhs.is_const():
                raise NotAffine("division by an index expression")
            return self.floordiv(lhs, rhs.const) if op == "//" else self.mod(lhs, rhs.const)
        raise NotAffine(f"operator `{op}` in an index expression")

    def rewrite(self, expr, substitution):
        """Replaces variables by expressions and re-normalises."""
        result = Affine(expr.const)
        for atom, coef in expr.terms.items():
            if atom[0] == "var":
                replacement = substitution.get(atom[1])
                result = result + (replacement if replacement is not None else Affine.var(atom[1])) * coef
            else:
                inner = self.rewrite(Affine.from_key(atom[1]), substitution)
                rebuilt = self.floordiv(inner, atom[2]) if atom[0] == "div" else self.mod(inner, atom[2])
                result = result + rebuilt * coef
        return result

    def fuse(self, exprs, outer, inner, block, fused):
        """Rewrites ``block * outer + inner`` as the single variable ``fused``.

        ``exprs`` may depend on ``outer`` and ``inner`` only through that
        combination; raises :class:`NotAffine` otherwise.  Returns the
        rewritten expressions; ``fused`` gets the combined range."""

        o_lo, o_hi = self.bounds.get(outer, (0, 0))
        i_lo, i_hi = self.bounds.get(inner, (0, 0))
        if i_hi - i_lo + 1 > block and o_hi > o_lo:
            raise NotAffine("tiles overlap")
        self.bounds[fused] = (block * o_lo + i_lo, block * o_hi + i_hi)
        if o_lo == o_hi:  # a single tile: the outer index is a constant
            substitution = {outer: Affine(o_lo), inner: Affine.var(fused) - block * o_lo}
            return [self.rewrite(expr, substitution) for expr in exprs]
        if i_lo == i_hi and block == 1:  # tiles of one element: the outer index is the coordinate
            substitution = {outer: Affine.var(fused) - i_lo, inner: Affine(i_lo)}
            return [self.rewrite(expr, substitution) for expr in exprs]

        marker = "ninetoothed_fuse_probe"

        def rewrite(expr):
            # substitute outer -> probe and inner -> fused - block * probe: the result is free of
            # the probe iff expr depends on the pair only through block * outer + inner
            substitution = {outer: Affine.var(marker), inner: Affine.var(fused) - Affine.var(marker) * block}
            wide = self.copy()
            wide.bounds[marker] = (o_lo, o_hi)
            rewritten = wide.rewrite(expr, substitution)
            if marker in rewritten.variables():
                raise NotAffine(f"`{outer}` and `{inner}` do not combine into one coordinate")
            return self.rewrite(rewritten, {})

        return [rewrite(expr) for expr in exprs]
