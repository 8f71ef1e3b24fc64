"""Ahead-of-time packaging: ``make(..., caller="hip", kernel_name=..., output_dir=...)``.

The reference's AOT path compiles the generated Triton kernel to a C source
and header that export ``launch_<kernel_name>(stream, tensors...)`` and builds
a shared library from them (src/ninetoothed/aot.py:23-106, 524-586, 802-898);
downstream C / C++ code links that library, and the returned Python handle
calls it through ctypes.  Here the kernels already exist in ``libnt_hip.so``,
so the package is a dispatcher: ``<kernel_name>.h`` declares
``launch_<kernel_name>`` with the reference's signature (one
``NineToothedTensor`` by value per application parameter, scalars as
zero-dimensional tensors), ``<kernel_name>.c`` forwards to the library entry
point of the recognised program with the element type and block sizes fixed at
packaging time, and ``<kernel_name>.so`` is built from it and linked against
``libnt_hip.so``.

Element-wise and reducing programs (tile maps) are lowered from the sizes of a call
(``ninetoothed_amd.mapping``).  For a package that lowering runs once, on sample sizes that
remember how every number was computed (``ninetoothed_amd.symbolic_int``): the C launch
function holds the lowered ``NineToothedMapProgram`` as a constant, checks the recorded
decisions against the sizes it is called with (returning 1, "no kernel", when one comes out
differently), recomputes the size-dependent fields and calls ``launch_nt_map``.  Declared
sizes (``Tensor(shape=(4096,))``) are plain numbers: nothing is left to check but the sizes.
"""

import ctypes
import pathlib
import shutil
import subprocess

from ninetoothed_amd import recognition, runtime
from ninetoothed_amd.recognition import UnsupportedProgram
from ninetoothed_amd.tensor import Tensor

INCLUDE_DIR = pathlib.Path(__file__).resolve().parent.parent / "include"

_ENUM_NAMES = {
    "i8": "NINETOOTHED_INT8", "i16": "NINETOOTHED_INT16", "i32": "NINETOOTHED_INT32", "i64": "NINETOOTHED_INT64",
    "u8": "NINETOOTHED_UINT8", "u16": "NINETOOTHED_UINT16", "u32": "NINETOOTHED_UINT32", "u64": "NINETOOTHED_UINT64",
    "fp16": "NINETOOTHED_FLOAT16", "bf16": "NINETOOTHED_BFLOAT16", "fp32": "NINETOOTHED_FLOAT32", "fp64": "NINETOOTHED_FLOAT64",
}


def _element_type(tensor, what):
    source = tensor.source
    dtype = source.dtype if isinstance(source.dtype, str) else None
    if dtype is None:
        current = tensor
        while isinstance(current.dtype, Tensor):
            current = current.dtype
        dtype = current.dtype if isinstance(current.dtype, str) else None
    if dtype not in _ENUM_NAMES:
        raise UnsupportedProgram(f"Ahead-of-time packaging needs the element type of `{what}`: pass `Tensor(..., dtype=ninetoothed.float16)`.")
    return dtype


def _probe_environment(kernel, sizes):
    """An environment with concrete, contiguous shapes for the structural check."""
    env = {}
    for tensor, shape in zip(kernel.types, sizes):
        if shape is None:
            continue
        source = tensor.source
        stride = 1
        strides = []
        for extent in reversed(shape):
            strides.insert(0, stride)
            stride *= extent
        for dim, extent in enumerate(shape):
            declared = source.shape[dim]
            if hasattr(declared, "is_name") and declared.is_name:
                env[declared.name] = extent
            env[source.size_string(dim)] = extent
            env[source.stride_string(dim)] = strides[dim]
    for name in kernel.meta_symbols:
        env.setdefault(name, 1)
    return env


def _conv2d_sample_sizes(kernel, constexprs):
    """Sample x[N,C,H,W], w[K,C,R,S], y[N,K,P,Q]: declared sizes where the tensors fix them."""

    def declared(tensor, defaults):
        return [int(size) if not hasattr(size, "is_name") else default for size, default in zip(tensor.source.shape, defaults)]

    n, c, h, w = declared(kernel.types[0], (2, 8, 10, 12))
    k, _, r, s = declared(kernel.types[1], (16, c, 3, 3))
    pad_h, pad_w = int(constexprs.get("padding_h", 0)), int(constexprs.get("padding_w", 0))
    return (n, c, h, w), (k, c, r, s), (n, k, h + 2 * pad_h - r + 1, w + 2 * pad_w - s + 1)


def _check_structure(kernel, constexprs):
    """Runs the call-time arrangement analysis on sample sizes: the dispatcher forwards whole
    tensors, which is only right if the arrangement is the program's canonical one."""
    kind = kernel.kind
    if kind == "matmul" and kernel.types[0].source.ndim == 4:
        sizes = _conv2d_sample_sizes(kernel, constexprs)
        env = _probe_environment(kernel, sizes)
        env.update(constexprs)
        result, info = recognition.analyze_gemm(kernel.types[0], kernel.types[1], kernel.types[2], env)
        if result != "conv2d":
            raise UnsupportedProgram("The arrangement is not the implicit-GEMM view of a convolution the packaged dispatcher forwards.")
        return {"conv2d": True, "pad_h": info["pad_h"], "pad_w": info["pad_w"], **info["blocks"]}
    if kind == "matmul" and kernel.types[0].source.ndim == 3:
        raise UnsupportedProgram("Batched products are not packaged ahead of time (call them through `make`).")
    if kind in ("matmul", "addmm"):
        m, n, k = 96, 160, 224
        if kind == "matmul":
            sizes = ((m, k), (k, n), (m, n))
            env = _probe_environment(kernel, sizes)
            env.update(constexprs)
            result, info = recognition.analyze_gemm(kernel.types[0], kernel.types[1], kernel.types[2], env)
        else:
            sizes = ((m, n), (m, k), (k, n), None, None, (m, n))
            env = _probe_environment(kernel, sizes)
            env.update(constexprs)
            result, info = recognition.analyze_gemm(kernel.types[1], kernel.types[2], kernel.types[5], env, input_type=kernel.types[0])
        if result != "strided" or (info["m"], info["n"], info["k"]) != (m, n, k):
            raise UnsupportedProgram("The arrangement is not the plain tiling of whole matrices the packaged dispatcher forwards.")
        return info["blocks"]
    if kind == "softmax":
        sizes = ((24, 200), (24, 200))
        env = _probe_environment(kernel, sizes)
        env.update(constexprs)
        for name in recognition.unbound_meta_symbols(kernel.types):
            env.setdefault(name, 1)
        missing = {"BLOCK_SIZE": 200}
        for name, value in missing.items():
            env.setdefault(name, value)
        recognition.analyze_softmax(kernel.types[0], kernel.types[1], env)
        return {}
    if kind == "attention":
        shape = (2, 3, 160, 64)
        scaled = kernel.details["scale"]
        sizes = (shape, shape, shape, None) + ((None,) if scaled else ()) + (shape,)
        env = _probe_environment(kernel, sizes)
        env.update(constexprs)
        o_type = kernel.types[5] if scaled else kernel.types[4]
        recognition.analyze_attention(kernel.types[0], kernel.types[1], kernel.types[2], o_type, env)
        return {}
    raise UnsupportedProgram(f"Programs of kind `{kind}` cannot be packaged ahead of time.")


# sample sizes for dimensions that are only known at launch, innermost first: odd, so that no
# tile size divides them (bounds checks stay in), and pairwise different
_SAMPLE_SIZES = (1000003, 1009, 101, 11, 7, 5, 3, 3)


def _c_double(value):
    if value != value:
        return "NAN"
    if value in (float("inf"), float("-inf")):
        return "INFINITY" if value > 0 else "-INFINITY"
    return float(value).hex()


def _c_initialiser(structure, indent="    "):
    """A ctypes structure as a C designated initialiser (zero fields and array tails left out)."""
    parts = []
    for field, kind in structure._fields_:
        value = getattr(structure, field)
        if isinstance(value, ctypes.Array):
            items = list(value)
            if items and isinstance(items[0], ctypes.Structure):
                texts = [_c_initialiser(item, indent + "    ") for item in items]
                while texts and texts[-1] == "{0}":
                    texts.pop()
            else:
                while items and items[-1] == 0 and not (isinstance(items[-1], float) and str(items[-1]) == "-0.0"):
                    items.pop()
                texts = [_c_double(item) if isinstance(item, float) else str(item) for item in items]
            if texts:
                parts.append(f".{field} = {{{', '.join(texts)}}}")
        elif isinstance(value, float):
            if value != 0 or str(value) == "-0.0":
                parts.append(f".{field} = {_c_double(value)}")
        elif value:
            parts.append(f".{field} = {value}")
    if not parts:
        return "{0}"
    return "{" + ", ".join(parts) + "}"


_FLOAT_TAGS = ("fp16", "bf16", "fp32", "fp64")


class MapPackage:
    """A tile-map program lowered on sample sizes: the programs, the size expressions of their
    call-dependent fields, and the decisions (guards) under which they hold."""

    def __init__(self, kernel, constexprs):
        from ninetoothed_amd import mapping
        from ninetoothed_amd.symbol import Symbol
        from ninetoothed_amd.symbolic_int import Recorder, SymInt

        self.parameters = list(kernel.parameters)
        self.declared = []       # (parameter, dimension, size) fixed by the tensors' declarations
        self.scalar_dtypes = {}  # parameter position -> element type of a call-time scalar
        self.ranks = [tensor.source.ndim for tensor in kernel.types]
        env, tags, sample_args = {}, {}, []
        # a dimension some tensor declares is the sample for the undeclared ones at the same place
        # (counted from the innermost), so that tensors of one shape stay of one shape
        samples = {}
        for tensor in kernel.types:
            for dim, declared in enumerate(tensor.source.shape):
                if not isinstance(declared, Symbol):
                    samples.setdefault(tensor.source.ndim - 1 - dim, int(declared))
        for position, (parameter, tensor) in enumerate(zip(self.parameters, kernel.types)):
            source = tensor.source
            if tensor.ndim == 0 and not isinstance(tensor.dtype, Tensor):
                if tensor.constexpr:
                    raise UnsupportedProgram("Compile-time scalars of a packaged element-wise program are not supported: declare a plain `Tensor(0)`.")
                declared = source.dtype if isinstance(source.dtype, str) else "fp64"
                if declared not in _ENUM_NAMES:
                    raise UnsupportedProgram(f"Scalar `{parameter}` has no packaged representation for type `{declared}`.")
                self.scalar_dtypes[position] = declared
                sample_args.append(1.0 if declared in _FLOAT_TAGS else 1)
                continue
            if source.jagged_dim is not None:
                raise UnsupportedProgram("Jagged tensors cannot be packaged ahead of time.")
            tags[position] = _element_type(tensor, parameter)
            sample_args.append(None)
            shape, sample_shape = [], []
            for dim, declared in enumerate(source.shape):
                if isinstance(declared, Symbol):
                    sample = samples.get(source.ndim - 1 - dim, _SAMPLE_SIZES[source.ndim - 1 - dim])
                    shape.append(SymInt.symbol(f"{parameter}.shape[{dim}]", sample))
                else:
                    sample = int(declared)
                    shape.append(sample)
                    self.declared.append((parameter, dim, sample))
                sample_shape.append(sample)
            stride = 1
            for dim in reversed(range(source.ndim)):
                env[source.stride_string(dim)] = SymInt.symbol(f"{parameter}.strides[{dim}]", stride)
                stride *= sample_shape[dim]
            for dim, declared in enumerate(source.shape):
                if isinstance(declared, Symbol) and declared.is_name:
                    env[declared.name] = shape[dim]
                env[source.size_string(dim)] = shape[dim]
        env.update(constexprs)
        for symbol in kernel.meta_symbols:
            env.setdefault(symbol, 1)

        with Recorder() as recorder:
            self.launches = []  # (program, scalar slots, operand parameters)
            for store in kernel.program.stores:
                built = mapping.build(store, kernel.types, sample_args, env, lambda p: tags[p], lambda p: 0, self.scalar_dtypes)
                if built is None:
                    raise UnsupportedProgram("The sample sizes give an empty launch: the program cannot be packaged.")
                program, _, scalar_slots, operand_params = built
                if any(isinstance(param, tuple) for param in operand_params):
                    raise UnsupportedProgram("Jagged tensors cannot be packaged ahead of time.")
                self.launches.append((program, scalar_slots, operand_params))
        self.guards = dict(recorder.guards)

    def instantiate(self, shapes, strides, scalars):
        """What the packaged C code computes for one call, in Python: the list of programs (data
        pointers left at zero), or ``None`` when a declared size or a guard does not hold.
        ``shapes`` / ``strides`` / ``scalars``: by parameter name."""
        from ninetoothed_amd import mapping
        from ninetoothed_amd.symbolic_int import evaluate, holds

        if any(shapes[parameter][dim] != size for parameter, dim, size in self.declared):
            return None
        if any(size == 0 for shape in shapes.values() for size in shape):
            return []  # an empty tensor: nothing to launch, like the launch-time path
        symbols = {}
        for parameter, shape in shapes.items():
            for dim, size in enumerate(shape):
                symbols[f"{parameter}.shape[{dim}]"] = size
                symbols[f"{parameter}.strides[{dim}]"] = strides[parameter][dim]
        for key, outcome in self.guards.items():
            if not holds(key, outcome, symbols):
                return None
        programs = []
        for template, scalar_slots, _ in self.launches:
            program = mapping.MapProgram.from_buffer_copy(bytes(template))
            for field, value in template.patches:
                name, index = field[:-1].split("[")
                getattr(program, name)[int(index)] = evaluate(value.expr, symbols)
            for index, param in scalar_slots:
                program.value_constants[index] = float(scalars[self.parameters[param]])
            programs.append(program)
        return programs

    def c_source(self, name):
        """Header and source of ``launch_<name>``."""
        from ninetoothed_amd.symbolic_int import C_HELPERS, CWriter

        parameters = self.parameters
        writer = CWriter()
        body = []
        if self.declared:
            body.append("/* sizes the tensors were declared with */")
            checks = " || ".join(f"{parameter}.shape[{dim}] != {size}ULL" for parameter, dim, size in self.declared)
            body.append(f"if ({checks})\n        return 1;")
        empty = " || ".join(
            f"{parameter}.shape[{dim}] == 0" for position, parameter in enumerate(parameters) if position not in self.scalar_dtypes
            for dim in range(self.ranks[position])
        )
        if empty:
            body.append("/* an empty tensor: nothing to launch */")
            body.append(f"if ({empty})\n        return 0;")
        if self.guards:
            body.append("/* decisions the lowering took on its sample sizes: the programs below hold for calls that repeat them */")
        for key, outcome in self.guards.items():
            failure = writer.failure(key, outcome)
            body.extend(writer.take_lines())
            body.append(f"if ({failure})\n        return 1;")
        templates = []
        for number, (program, scalar_slots, operand_params) in enumerate(self.launches):
            templates.append(f"static const NineToothedMapProgram {name}_program_{number} = {_c_initialiser(program)};")
            block = [f"NineToothedMapProgram program = {name}_program_{number};"]
            for field, value in program.patches:
                text = writer.value(value.expr)
                body.extend(writer.take_lines())
                block.append(f"program.{field} = {'(double)' if field.startswith('value_constants') else ''}{text};")
            for slot, param in enumerate(operand_params):
                block.append(f"program.operands[{slot}].data = {parameters[param]}.data;")
            for index, param in scalar_slots:
                read = "*(const double *)" if self.scalar_dtypes[param] in _FLOAT_TAGS else "(double)*(const int64_t *)"
                block.append(f"program.value_constants[{index}] = {read}{parameters[param]}.data;")
            block.append("NineToothedResult result = launch_nt_map(stream, &program);")
            block.append("if (result != 0)\n            return result;")
            body.append("{\n        " + "\n        ".join(block) + "\n    }")
        body.append("return 0;")

        arguments = ", ".join(f"NineToothedTensor {parameter}" for parameter in parameters)
        signature = f"NineToothedResult launch_{name}(NineToothedStream stream, {arguments})"
        header = (
            f"/* launch_{name}: packaged element-wise program ({len(self.launches)} launch(es) of launch_nt_map in libnt_hip.so). */\n"
            f"#ifndef NINETOOTHED_{name.upper()}_H\n#define NINETOOTHED_{name.upper()}_H\n\n"
            '#include "ninetoothed_hip.h"\n\n#ifdef __cplusplus\nextern "C" {\n#endif\n\n'
            f"{signature};\n\n#ifdef __cplusplus\n}}\n#endif\n\n#endif\n"
        )
        source = (
            f'#include "{name}.h"\n\n#include <math.h>\n#include <stdint.h>\n\n' + C_HELPERS + "\n" + "\n".join(templates)
            + f"\n\n{signature} {{\n    " + "\n    ".join(body) + "\n}\n"
        )
        return header, source


def _dispatcher_source(kernel, name, dtype, out_dtype, blocks):
    parameters = ", ".join(f"NineToothedTensor {parameter}" for parameter in kernel.parameters)
    signature = f"NineToothedResult launch_{name}(NineToothedStream stream, {parameters})"
    p = kernel.parameters
    bm, bn, bk = (blocks.get(axis, 0) if blocks.get(axis, 0) > 1 else 0 for axis in ("m", "n", "k"))
    if blocks.get("conv2d"):
        body = f"return launch_nt_conv2d(stream, {p[0]}, {p[1]}, {p[2]}, {_ENUM_NAMES[dtype]}, {blocks['pad_h']}, {blocks['pad_w']}, {bm}, {bn}, {bk});"
    elif kernel.kind == "matmul":
        body = f"return launch_nt_matmul(stream, {p[0]}, {p[1]}, {p[2]}, {_ENUM_NAMES[dtype]}, {_ENUM_NAMES[out_dtype]}, {bm}, {bn}, {bk});"
    elif kernel.kind == "addmm":
        body = f"return launch_nt_addmm(stream, {p[0]}, {p[1]}, {p[2]}, {p[3]}, {p[4]}, {p[5]}, {_ENUM_NAMES[dtype]}, {bm}, {bn}, {bk});"
    elif kernel.kind == "softmax":
        body = f"return launch_nt_softmax(stream, {p[0]}, {p[1]}, {_ENUM_NAMES[dtype]}, {p[0]}.shape ? (int){p[0]}.shape[1] : 0);"
    else:
        if kernel.details["scale"]:
            body = f"return launch_nt_attention(stream, {p[0]}, {p[1]}, {p[2]}, {p[3]}, {p[4]}, {p[5]}, {_ENUM_NAMES[dtype]}, 0, 0);"
        else:
            body = (
                "NineToothedTensor no_scale = {0, 0, 0};\n"
                f"    return launch_nt_attention(stream, {p[0]}, {p[1]}, {p[2]}, {p[3]}, no_scale, {p[4]}, {_ENUM_NAMES[dtype]}, 0, 0);"
            )
    header = (
        f"/* launch_{name}: packaged `{kernel.kind}` program (element type {dtype}); forwards to libnt_hip.so. */\n"
        f"#ifndef NINETOOTHED_{name.upper()}_H\n#define NINETOOTHED_{name.upper()}_H\n\n"
        '#include "ninetoothed_hip.h"\n\n#ifdef __cplusplus\nextern "C" {\n#endif\n\n'
        f"{signature};\n\n#ifdef __cplusplus\n}}\n#endif\n\n#endif\n"
    )
    source = f'#include "{name}.h"\n\n{signature} {{\n    {body}\n}}\n'
    return header, source


def generate(arrangement, application, tensors, kernel_name, output_dir, constexprs=None, block_hints=True):
    """Writes ``<kernel_name>.h`` and ``<kernel_name>.c`` and returns the analysed kernel.

    With ``block_hints=False`` the dispatcher passes no block sizes, which leaves the choice of
    the GEMM instance to the library (its heuristic table and tuning cache)."""
    from ninetoothed_amd.make import Kernel

    if kernel_name is None or output_dir is None:
        raise ValueError("Ahead-of-time packaging needs `kernel_name` and `output_dir`.")
    types = arrangement(*tensors)
    types = types if isinstance(types, tuple) else (types,)
    kernel = Kernel(application, types, kernel_name=kernel_name)
    output_dir = pathlib.Path(output_dir)
    if kernel.kind == "map":
        kernel.map_package = MapPackage(kernel, dict(constexprs or {}))
        header, source = kernel.map_package.c_source(kernel_name)
        output_dir.mkdir(parents=True, exist_ok=True)
        (output_dir / f"{kernel_name}.h").write_text(header)
        (output_dir / f"{kernel_name}.c").write_text(source)
        return kernel
    blocks = _check_structure(kernel, dict(constexprs or {}))
    if not block_hints:
        blocks = {name: value for name, value in blocks.items() if name not in ("m", "n", "k")}
    tensor_types = [t for t in kernel.types if not (t.ndim == 0 and not isinstance(t.dtype, Tensor))]
    dtype = _element_type(tensor_types[0], kernel.parameters[0])
    out_dtype = _element_type(tensor_types[-1], kernel.parameters[-1])
    for tensor in tensor_types[:-1]:
        if _element_type(tensor, "an operand") != dtype:
            raise UnsupportedProgram("Operands of a packaged kernel must share one element type.")
    header, source = _dispatcher_source(kernel, kernel_name, dtype, out_dtype, blocks)
    output_dir.mkdir(parents=True, exist_ok=True)
    (output_dir / f"{kernel_name}.h").write_text(header)
    (output_dir / f"{kernel_name}.c").write_text(source)
    return kernel


def compile_library(sources, library, include_dirs):
    """Builds a shared library from C sources, linked against ``libnt_hip.so``."""
    compiler = shutil.which("gcc") or shutil.which("cc") or shutil.which("hipcc")
    if compiler is None:
        raise RuntimeError("No C compiler found to build the packaged kernel.")
    lib_dir = runtime.LIBRARY_PATH.parent
    command = [
        compiler, "-shared", "-fPIC", "-O2", f"-I{INCLUDE_DIR}", *(f"-I{path}" for path in include_dirs), *map(str, sources),
        f"-L{lib_dir}", "-lnt_hip", f"-Wl,-rpath,{lib_dir}", "-o", str(library),
    ]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError("Building the packaged kernel failed:\n" + " ".join(command) + "\n" + result.stderr)
    return library


def package(arrangement, application, tensors, kernel_name, output_dir, constexprs=None):
    """Writes ``<kernel_name>.h/.c``, builds ``<kernel_name>.so`` and returns a handle."""
    kernel = generate(arrangement, application, tensors, kernel_name, output_dir, constexprs)
    output_dir = pathlib.Path(output_dir)
    library = compile_library([output_dir / f"{kernel_name}.c"], output_dir / f"{kernel_name}.so", [output_dir])
    return PackagedKernel(library, kernel_name, kernel)


class PackagedKernel:
    """Calls ``launch_<kernel_name>`` of a packaged library with torch tensors, the way the
    reference's AOT handle does (src/ninetoothed/aot.py:802-862)."""

    def __init__(self, library_path, kernel_name, kernel):
        self.library_path = str(library_path)
        self.kernel_name = kernel_name
        self.kind = kernel.kind
        self._scalar = scalar_kinds(kernel)
        self._library = ctypes.CDLL(self.library_path)
        self._function = getattr(self._library, f"launch_{kernel_name}")
        self._function.argtypes = [ctypes.c_void_p] + [runtime.ArgumentTensor] * len(kernel.types)
        self._function.restype = ctypes.c_int
        self._source = str(pathlib.Path(self.library_path).with_suffix(".c"))

    def __call__(self, *args):
        if len(args) != len(self._scalar):
            raise TypeError(f"`{self.kernel_name}` takes {len(self._scalar)} arguments but {len(args)} were given.")
        runtime.check(self._function(runtime.current_stream(), *marshal(args, self._scalar)))


def scalar_kinds(kernel):
    """Per application parameter: ``None`` for a tensor, else how the launch function reads the
    zero-dimensional tensor -- ``"float"`` (a host double) or ``"int"`` (a host int64).  The
    declared element type decides (src/ninetoothed/aot.py:234-283, 610-630); undeclared scalars
    are doubles, except the causal flag of the attention program."""
    kinds = []
    for position, tensor in enumerate(kernel.types):
        if not (tensor.ndim == 0 and not isinstance(tensor.dtype, Tensor)):
            kinds.append(None)
        elif isinstance(tensor.source.dtype, str):
            kinds.append("float" if tensor.source.dtype in _FLOAT_TAGS else "int")
        else:
            kinds.append("int" if kernel.kind == "attention" and position == 3 else "float")
    return kinds


def marshal(args, scalar):
    """Torch tensors and Python scalars as the ``NineToothedTensor`` values a packaged launch function
    takes; ``scalar``: per argument ``None`` / ``False`` (a tensor), ``"float"``, ``"int"`` or ``True``
    (by the type of the Python value)."""
    import torch

    marshalled = []
    for arg, kind in zip(args, scalar):
        if kind:
            value = arg.item() if isinstance(arg, torch.Tensor) else arg
            is_float = isinstance(value, float) if kind is True else kind == "float"
            marshalled.append(runtime.ArgumentTensor.from_scalar(float(value) if is_float else int(value)))
        else:
            if not arg.is_cuda:
                raise RuntimeError("Packaged kernels run on the GPU only (there is no CPU path).")
            marshalled.append(runtime.ArgumentTensor.from_torch_tensor(arg))
    return marshalled
