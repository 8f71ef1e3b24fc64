"""The ``ntl`` namespace applications are written against.

In the reference every ``ntl.X`` is rewritten textually to
``triton.language.X`` (src/ninetoothed/language.py:1-26,
src/ninetoothed/generation.py:849-855).  Here an application is never executed
as Python: it is traced into a dataflow graph (:mod:`ninetoothed_amd.tracing`),
and the names below only have to exist so that user modules import cleanly and
the tracer can tell which function or dtype a name denotes.
"""

from ninetoothed_amd import dtype as _dtype


class _Function:
    """A device-side function known to the tracer."""

    def __init__(self, name):
        self.name = name

    def __call__(self, *args, **kwargs):
        raise RuntimeError(
            f"`ntl.{self.name}` only has a meaning inside an application passed to `ninetoothed_amd.make` or `jit`."
        )

    def __repr__(self):
        return f"ntl.{self.name}"


_FUNCTIONS = (
    "zeros",
    "full",
    "dot",
    "trans",
    "max",
    "min",
    "sum",
    "maximum",
    "minimum",
    "exp",
    "exp2",
    "log",
    "log2",
    "sqrt",
    "rsqrt",
    "abs",
    "where",
    "cast",
    "sigmoid",
    "softmax",
    "arange",
    "program_id",
    "rand",
    "cdiv",
    "sin",
    "cos",
    "floor",
    "ceil",
    "load",
    "store",
    "atomic_add",
)

for _name in _FUNCTIONS:
    globals()[_name] = _Function(_name)


class _LibDevice:
    """``ninetoothed.language.libdevice``: math functions by name
    (src/ninetoothed/language.py:1-26 re-exports Triton's ``libdevice``)."""

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        return _Function("libdevice." + name)


libdevice = _LibDevice()

int8 = _dtype.int8
int16 = _dtype.int16
int32 = _dtype.int32
int64 = _dtype.int64
uint8 = _dtype.uint8
uint16 = _dtype.uint16
uint32 = _dtype.uint32
uint64 = _dtype.uint64
float16 = _dtype.float16
bfloat16 = _dtype.bfloat16
float32 = _dtype.float32
float64 = _dtype.float64


def is_function(value):
    return isinstance(value, _Function)
