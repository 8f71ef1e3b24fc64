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

Only the recognised programs (matmul, addmm, softmax, attention, conv2d) can be packaged: tile maps are lowered per
call from the sizes of the arguments (``ninetoothed_amd.mapping``), which a C
dispatcher cannot do.
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
    output_dir = pathlib.Path(output_dir)
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
        self._scalar = [t.ndim == 0 and not isinstance(t.dtype, Tensor) for t in kernel.types]
        self._library = ctypes.CDLL(self.library_path)
        self._function = getattr(self._library, f"launch_{kernel_name}")
        self._function.argtypes = [ctypes.c_void_p] + [runtime.ArgumentTensor] * len(kernel.types)
        self._function.restype = ctypes.c_int
        self._source = str(pathlib.Path(self.library_path).with_suffix(".c"))

    def __call__(self, *args):
        if len(args) != len(self._scalar):
            raise TypeError(f"`{self.kernel_name}` takes {len(self._scalar)} arguments but {len(args)} were given.")
        runtime.check(self._function(runtime.current_stream(), *marshal(args, self._scalar)))


def marshal(args, scalar):
    """Torch tensors and Python scalars as the ``NineToothedTensor`` values a packaged launch function takes."""
    import torch

    marshalled = []
    for arg, is_scalar in zip(args, scalar):
        if is_scalar:
            value = arg.item() if isinstance(arg, torch.Tensor) else arg
            marshalled.append(runtime.ArgumentTensor.from_scalar(float(value) if isinstance(value, float) else int(value)))
        else:
            if not arg.is_cuda:
                raise RuntimeError("Packaged kernels run on the GPU only (there is no CPU path).")
            marshalled.append(runtime.ArgumentTensor.from_torch_tensor(arg))
    return marshalled
