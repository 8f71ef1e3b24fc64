"""``build(premake, configs, ...)``: one library that dispatches over several configurations.

Mirrors the reference's ``ninetoothed.build`` (src/ninetoothed/build.py:26-213): every
configuration ``(args, kwargs, compilation_configs)`` is turned into a kernel by
``premake(*args, **kwargs) -> (arrangement, application, tensors)``, packaged as
``launch_<kernel_name>_<values>``, and ``<kernel_name>.h/.c`` export::

    NineToothedResult launch_<kernel_name>(NineToothedStream stream,
                                           NineToothedTensor <application parameters>...,
                                           int <premake parameter>_..., int <compilation config>...);

which compares the trailing integers with each configuration (dtypes as ``NineToothedDataType``
values, ``None`` and ``False`` as 0, ``True`` as 1 -- ``_arg_to_int``, build.py:799-812) and
returns 1 when none matches (build.py:134-170).

``meta_parameters`` names premake parameters that only steer performance (block sizes).  The
reference times every value of them per remaining configuration and emits a dispatcher
without those parameters (build.py:180-211, 363-455).  Here block sizes are hints that pick
among the library's GEMM instances, and the library owns that choice (heuristic table, the
first-launch tuner and its CSV cache), so with ``meta_parameters`` the dispatcher drops them
from the signature and the packaged kernels pass no block hint at all.

A fingerprint of the premake source, the configurations and the library version is kept in
``<kernel_name>.fingerprint`` (build.py:617-660); an unchanged fingerprint reuses the built
library.  ``lazy=True`` postpones all of this to the first call (build.py:222-233).
"""

import ctypes
import functools
import hashlib
import inspect
import pathlib

from ninetoothed_amd import aot, runtime
from ninetoothed_amd.tensor import Tensor


def _arg_to_int(value):
    if type(value) is int:
        return value
    if value is None or isinstance(value, bool):
        return int(bool(value))
    if isinstance(value, str) and value in runtime.DATA_TYPE_INDEX:
        return runtime.DATA_TYPE_INDEX[value]
    raise TypeError(f"Configuration value {value!r} cannot be passed to a C dispatcher as an integer.")


def _fingerprint(premake, configs, meta_parameters, caller):
    hasher = hashlib.sha256()
    target = premake.func if isinstance(premake, functools.partial) else premake
    try:
        hasher.update(inspect.getsource(target).encode())
    except (TypeError, OSError):
        hasher.update(repr(target).encode())
    if isinstance(premake, functools.partial):
        hasher.update(repr((premake.args, sorted(premake.keywords.items()))).encode())
    hasher.update(repr((configs, meta_parameters, caller)).encode())
    for path in (pathlib.Path(__file__), pathlib.Path(aot.__file__)):
        hasher.update(path.read_bytes())
    return hasher.hexdigest()


class _Configuration:
    def __init__(self, premake, config, meta_parameters):
        args, kwargs, compilation_configs = config
        self.arrangement, self.application, self.tensors = premake(*args, **kwargs)
        bound = inspect.signature(premake).bind(*args, **kwargs)
        bound.apply_defaults()
        self.combination = {f"{name}_": _arg_to_int(value) for name, value in bound.arguments.items()}
        self.combination.update({name: _arg_to_int(value) for name, value in compilation_configs.items()})
        # meta parameters: the named premake parameters and, when any are named, every compilation config
        self.meta = {f"{name}_" for name in meta_parameters if name in bound.arguments}
        if meta_parameters:
            self.meta.update(compilation_configs)
        self.parameters = tuple(inspect.signature(self.application).parameters)

    def key(self, without_meta):
        return {name: value for name, value in self.combination.items() if not (without_meta and name in self.meta)}


def _build(premake, configs, meta_parameters, caller, kernel_name, output_dir):
    output_dir = pathlib.Path(output_dir)
    output_dir.mkdir(parents=True, exist_ok=True)
    library = output_dir / f"{kernel_name}.so"
    fingerprint_path = output_dir / f"{kernel_name}.fingerprint"
    fingerprint = _fingerprint(premake, configs, meta_parameters, caller)
    tuned = meta_parameters is not None
    meta_names = tuple(meta_parameters or ())

    configurations = [_Configuration(premake, config, meta_names) for config in configs]
    if not configurations:
        raise ValueError("`build` needs at least one configuration.")

    # configurations that differ only in meta parameters collapse into one packaged kernel
    branches = {}
    for configuration in configurations:
        key = configuration.key(without_meta=tuned)
        branches.setdefault(tuple(key.items()), configuration)

    tensor_parameters = max((c.parameters for c in configurations), key=len)
    config_parameters = tuple(dict.fromkeys(name for key in branches for name, _ in key))
    # scalars travel as host doubles / int64s: by the declared element type, else by the Python value's type
    scalar = [
        (("float" if t.dtype in aot._FLOAT_TAGS else "int") if isinstance(t.dtype, str) else True) if t.ndim == 0 and not isinstance(t.dtype, Tensor) else None
        for t in configurations[0].tensors
    ]

    if not (library.exists() and fingerprint_path.exists() and fingerprint_path.read_text().strip() == fingerprint):
        sources, includes, launches = [], [], []
        for key, configuration in branches.items():
            name = f"{kernel_name}_" + "_".join(str(value).replace("-", "n") for _, value in key)
            aot.generate(configuration.arrangement, configuration.application, configuration.tensors, name, output_dir, block_hints=not tuned)
            sources.append(output_dir / f"{name}.c")
            includes.append(f'#include "{name}.h"')
            condition = " && ".join(f"{parameter} == {value}" for parameter, value in key) or "1"
            arguments = ", ".join(("stream",) + configuration.parameters)
            launches.append(f"    if ({condition})\n        return launch_{name}({arguments});")
        declarations = ", ".join(
            ["NineToothedStream stream"] + [f"NineToothedTensor {name}" for name in tensor_parameters] + [f"int {name}" for name in config_parameters]
        )
        signature = f"NineToothedResult launch_{kernel_name}({declarations})"
        header = (
            f"/* launch_{kernel_name}: dispatches over {len(branches)} packaged configuration(s); returns 1 when none matches. */\n"
            f"#ifndef NINETOOTHED_{kernel_name.upper()}_H\n#define NINETOOTHED_{kernel_name.upper()}_H\n\n"
            '#include "ninetoothed_hip.h"\n\n#ifdef __cplusplus\nextern "C" {\n#endif\n\n'
            f"{signature};\n\n#ifdef __cplusplus\n}}\n#endif\n\n#endif\n"
        )
        source = f'#include "{kernel_name}.h"\n\n' + "\n".join(includes) + f"\n\n{signature} {{\n" + "\n".join(launches) + "\n    return 1;\n}\n"
        (output_dir / f"{kernel_name}.h").write_text(header)
        (output_dir / f"{kernel_name}.c").write_text(source)
        aot.compile_library([output_dir / f"{kernel_name}.c", *sources], library, [output_dir])
        fingerprint_path.write_text(fingerprint)

    return BuiltKernel(library, kernel_name, scalar, config_parameters)


class BuiltKernel:
    """Calls ``launch_<kernel_name>(stream, tensors..., configuration values...)``."""

    def __init__(self, library_path, kernel_name, scalar, config_parameters):
        self.library_path = str(library_path)
        self.kernel_name = kernel_name
        self.config_parameters = config_parameters
        self._scalar = scalar
        self._library = ctypes.CDLL(self.library_path)
        self._function = getattr(self._library, f"launch_{kernel_name}")
        self._function.argtypes = [ctypes.c_void_p] + [runtime.ArgumentTensor] * len(scalar) + [ctypes.c_int] * len(config_parameters)
        self._function.restype = ctypes.c_int

    def __call__(self, *args):
        expected = len(self._scalar) + len(self.config_parameters)
        if len(args) != expected:
            raise TypeError(
                f"`{self.kernel_name}` takes {len(self._scalar)} tensors and {len(self.config_parameters)} configuration values "
                f"({', '.join(self.config_parameters)}) but {len(args)} arguments were given."
            )
        tensors = aot.marshal(args[: len(self._scalar)], self._scalar)
        values = [_arg_to_int(value) for value in args[len(self._scalar) :]]
        runtime.check(self._function(runtime.current_stream(), *tensors, *values))


class _LazyKernel:
    def __init__(self, factory):
        self._factory = factory
        self._kernel = None

    def __call__(self, *args):
        if self._kernel is None:
            self._kernel = self._factory()
        return self._kernel(*args)


def build(premake, configs, *, meta_parameters=None, caller="hip", kernel_name=None, output_dir=None, lazy=False):
    """Packages every configuration and returns a handle that calls the dispatcher."""
    if caller not in ("hip", "cuda"):
        raise ValueError(f"Unsupported caller `{caller}`: this package runs on the GPU only.")
    if kernel_name is None or output_dir is None:
        raise ValueError("`build` needs `kernel_name` and `output_dir`.")
    factory = functools.partial(_build, premake, tuple(configs), meta_parameters, caller, kernel_name, output_dir)
    return _LazyKernel(factory) if lazy else factory()
