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
from ninetoothed_amd.eval import _eval as eval  # noqa: A001  (the reference's public name, src/ninetoothed/__init__.py:16-17)
from ninetoothed_amd.eval import _subs as subs
from ninetoothed_amd.jit import jit  # (binds the decorator over the submodule of the same name, as the reference does)
from ninetoothed_amd.make import Kernel, make
from ninetoothed_amd.recognition import UnsupportedProgram
from ninetoothed_amd.runtime import KernelLaunchError
from ninetoothed_amd.symbol import Symbol, block_size
from ninetoothed_amd.tensor import Tensor


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
