"""The one thing of the reference's code generator that programs reach for from outside.

The reference generates Triton source per program (src/ninetoothed/generation.py:28-837) and
caches it under ``CACHE_DIR`` (``generation.py:24-25, 875``); its own ahead-of-time tests pass
that directory as ``output_dir`` (``tests/test_aot.py:37``: ``ninetoothed.generation.CACHE_DIR``).
This build generates no source -- programs are recognised and served by the kernels of
``libnt_hip.so`` -- so the module only provides that directory, for programs written against
the reference that name it.  It is created on first use, like the reference's.
"""

import os
import pathlib

CACHE_DIR = pathlib.Path(os.environ.get("NINETOOTHED_AMD_CACHE_DIR") or pathlib.Path.home() / ".ninetoothed_amd")
try:
    CACHE_DIR.mkdir(parents=True, exist_ok=True)
except OSError:  # a read-only home directory: the caller finds out when it writes
    pass
