"""The reference's import name for this build.

Programs written for ninetoothed start with ``import ninetoothed``,
``import ninetoothed.language as ntl`` or ``from ninetoothed import Tensor``
(README.md:30-34 and every test program of the reference).  This package holds
no code of its own: every name and every submodule *is* the corresponding
object of :mod:`ninetoothed_amd` (``ninetoothed.language is
ninetoothed_amd.language``), so kernels, tensors and exceptions made through
either name are interchangeable.
"""

import importlib
import importlib.abc
import importlib.util
import sys

import ninetoothed_amd
from ninetoothed_amd import *  # noqa: F401,F403
from ninetoothed_amd import __all__  # noqa: F401

_PREFIX = __name__ + "."
_TARGET = ninetoothed_amd.__name__ + "."


class _AliasLoader(importlib.abc.Loader):
    """Hands out the already imported ``ninetoothed_amd.<name>`` module object."""

    def __init__(self, target):
        self._target = target

    def create_module(self, spec):
        module = importlib.import_module(self._target)
        self._own_spec = module.__spec__
        return module

    def exec_module(self, module):
        # the module was executed under its own name; the import system has just pointed
        # its `__spec__` at the alias, which would misdirect `importlib.reload`
        module.__spec__ = self._own_spec


class _AliasFinder(importlib.abc.MetaPathFinder):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(_PREFIX):
            return None
        real = _TARGET + fullname[len(_PREFIX):]
        try:
            if importlib.util.find_spec(real) is None:
                return None
        except ModuleNotFoundError:
            return None
        return importlib.util.spec_from_loader(fullname, _AliasLoader(real))


if not any(isinstance(finder, _AliasFinder) for finder in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())

# `jit` and `eval` name a submodule AND a public function (src/ninetoothed/__init__.py:16-18 imports the functions
# over the submodules).  The first import of a submodule binds it in its parent package, so both are imported here
# once and the functions bound over them afterwards: a later `from ninetoothed.jit import jit` then finds the module
# in `sys.modules` and leaves `ninetoothed.jit` the decorator.
for _name in ("jit", "eval"):
    importlib.import_module(_PREFIX + _name)
jit = ninetoothed_amd.jit
eval = ninetoothed_amd.eval  # noqa: A001


def __getattr__(name):
    """``ninetoothed.<submodule>`` without an explicit import of the submodule."""
    try:
        module = importlib.import_module(_PREFIX + name)
    except ModuleNotFoundError:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}") from None
    return module
