"""Name mangling of the reference's code generator (src/ninetoothed/naming.py:4-54).

The reference marks what kind of thing a generated identifier stands for by
prefixing it: ``ninetoothed_constexpr_prefix_<name>`` for call-time constants,
``ninetoothed_meta_prefix_<name>`` for tunable meta-parameters (which are
constants as well) and ``ninetoothed_next_power_of_2_prefix_<name>`` for the
rounded-up inner extents of ``tl.arange``.  Prefixes stack.  This build keeps
those kinds as attributes of :class:`ninetoothed_amd.symbol.Symbol` and
generates no identifiers, so nothing on the launch path calls this module; it
is here for programs and tools that import ``ninetoothed.naming`` and must see
the same strings (``tests/test_naming.py`` of the reference).
"""

_HEAD = "ninetoothed_"
_TAIL = "_prefix_"
_KINDS = ("constexpr", "meta", "next_power_of_2")


def auto_generate(name):
    """The identifier the generator reserves for a helper of its own."""
    return _HEAD + name


def make_constexpr(name):
    return _wrap("constexpr", name)


def make_meta(name):
    return _wrap("meta", name)


def make_next_power_of_2(name):
    return _wrap("next_power_of_2", name)


def is_constexpr(name):
    """Meta-parameters are call-time constants too."""
    kinds = _kinds_of(name)
    return "constexpr" in kinds or "meta" in kinds


def is_meta(name):
    return "meta" in _kinds_of(name)


def is_next_power_of_2(name):
    return "next_power_of_2" in _kinds_of(name)


def remove_prefixes(name):
    """``name`` without any of the stacked kind prefixes."""
    return _split(name)[1]


def _wrap(kind, name):
    return f"{_HEAD}{kind}{_TAIL}{name}"


def _split(name):
    """The kinds of the prefixes that ``name`` starts with, outermost first, and the bare name."""
    kinds = []
    stripped = True
    while stripped:
        stripped = False
        for kind in _KINDS:
            prefix = _HEAD + kind + _TAIL
            if name.startswith(prefix):
                kinds.append(kind)
                name = name[len(prefix):]
                stripped = True
                break
    return kinds, name


def _kinds_of(name):
    return set(_split(name)[0])
