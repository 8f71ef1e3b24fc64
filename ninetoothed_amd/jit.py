"""``from ninetoothed.jit import jit``: the decorator form of ``make`` under the module name the
reference keeps it in (src/ninetoothed/jit.py:8-59).  The package attribute ``ninetoothed.jit``
is the decorator itself, as in the reference, whose ``__init__`` imports the function over the
submodule of the same name."""

from ninetoothed_amd.make import jit

__all__ = ["jit"]
