"""ninetoothed_amd: the arrange-and-apply programming surface of ninetoothed
(``Tensor``, ``Symbol``, ``block_size``, ``make``, ``jit``, ``ninetoothed_amd.language``)
executed by hand-written gfx950 (MI355X) kernels.

Public names follow the reference package (src/ninetoothed/__init__.py:1-44).
"""

from ninetoothed_amd.build import build
from ninetoothed_amd.dtype import (
    bfloat16,
    float16,
    float32,
    float64,
    int8,
    int16,
    int32,
    int64,
    uint8,
    uint16,
    uint32,
    uint64,
)
from ninetoothed_amd.make import Kernel, jit, make
from ninetoothed_amd.recognition import UnsupportedProgram
from ninetoothed_amd.runtime import KernelLaunchError
from ninetoothed_amd.symbol import Symbol, block_size
from ninetoothed_amd.tensor import Tensor


def eval(tensor, subs=None):
    """Evaluates a symbolic tensor (see :meth:`Tensor.eval`)."""
    return tensor.eval(subs)


def subs(tensor, substitutions):
    """Substitutes symbols in a tensor (see :meth:`Tensor.subs`)."""
    return tensor.subs(substitutions)


__all__ = [
    "Kernel",
    "KernelLaunchError",
    "Symbol",
    "Tensor",
    "UnsupportedProgram",
    "bfloat16",
    "block_size",
    "build",
    "eval",
    "float16",
    "float32",
    "float64",
    "int8",
    "int16",
    "int32",
    "int64",
    "jit",
    "make",
    "subs",
    "uint8",
    "uint16",
    "uint32",
    "uint64",
]
