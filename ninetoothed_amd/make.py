"""``make`` and ``jit``: bind an arrangement to an application and return a
callable on torch tensors.

Same surface as the reference (src/ninetoothed/make.py:7-56,
src/ninetoothed/jit.py:8-128): ``make(arrangement, application, tensors)`` runs
the arrangement on the symbolic tensors and pairs its results with the
application's parameters by position; ``jit`` takes them from the parameter
annotations.  The returned kernel is called with one argument per application
parameter, in order (torch tensors; Python numbers for zero-dimensional
tensors) plus the arrangement's call-time constants by keyword (for example
``BLOCK_SIZE=``, ``padding_h=``); it writes its outputs in place and returns
``None`` (launch convention: src/ninetoothed/generation.py:518-600).

Instead of generating and compiling code, the kernel object recognises the
program (:mod:`ninetoothed_amd.recognition`) and, per distinct combination of
shapes / strides / dtypes, prepares a launch plan for ``libnt_hip.so``.
"""

import hashlib
import inspect
import os
import pathlib

from ninetoothed_amd import recognition, runtime
from ninetoothed_amd.recognition import UnsupportedProgram
from ninetoothed_amd.symbol import Symbol
from ninetoothed_amd.tensor import Tensor

CACHE_DIR = pathlib.Path(os.environ.get("NINETOOTHED_AMD_CACHE_DIR") or pathlib.Path.home() / ".ninetoothed_amd")

_TORCH_DTYPE_TAGS = None


def _dtype_tag(torch_dtype):
    global _TORCH_DTYPE_TAGS
    if _TORCH_DTYPE_TAGS is None:
        import torch

        _TORCH_DTYPE_TAGS = {
            torch.int8: "i8",
            torch.int16: "i16",
            torch.int32: "i32",
            torch.int64: "i64",
            torch.uint8: "u8",
            torch.float16: "fp16",
            torch.bfloat16: "bf16",
            torch.float32: "fp32",
            torch.float64: "fp64",
            torch.bool: "u8",
        }
        if hasattr(torch, "float8_e5m2"):
            _TORCH_DTYPE_TAGS[torch.float8_e5m2] = "fp8e5m2"
    try:
        return _TORCH_DTYPE_TAGS[torch_dtype]
    except KeyError:
        raise UnsupportedProgram(f"Element type `{torch_dtype}` is not supported.") from None


def make(
    arrangement,
    application,
    tensors,
    caller="torch",
    kernel_name=None,
    output_dir=None,
    num_warps=None,
    num_stages=None,
    max_num_configs=None,
):
    """Integrates the arrangement and the application of the tensors.

    :param arrangement: The arrangement of the tensors.
    :param application: The application of the tensors.
    :param tensors: The tensors.
    :param caller: Who will call the compute kernel: ``"torch"``, or ``"hip"``
        (alias ``"cuda"``) to package the kernel ahead of time as
        ``<output_dir>/<kernel_name>.{h,c,so}`` exporting ``launch_<kernel_name>``.
    :param kernel_name: The name for the kernel.
    :param output_dir: Where the packaged files go (``"hip"`` only).
    :param num_warps: Accepted for compatibility; wave counts belong to the
        hand-written kernels.
    :param num_stages: Accepted for compatibility; see ``num_warps``.
    :param max_num_configs: Accepted for compatibility; tile selection is
        done inside the library.
    :return: A handle to the compute kernel.
    """

    if caller in ("hip", "cuda"):  # ahead-of-time packaging (the reference's `caller="cuda"`, src/ninetoothed/make.py:38-56)
        from ninetoothed_amd import aot

        return aot.package(arrangement, application, tensors, kernel_name, output_dir)
    if caller != "torch":
        raise NotImplementedError(f"Unknown caller `{caller}`: use \"torch\" or \"hip\".")
    types = arrangement(*tensors)
    types = types if isinstance(types, tuple) else (types,)
    return Kernel(application, types, kernel_name=kernel_name)


def jit(func=None, *, caller="torch", kernel_name=None, num_warps=None, num_stages=None, max_num_configs=None, _prettify=False):
    """A decorator that builds a kernel from a function whose parameter
    annotations are arranged tensors."""

    if caller != "torch":
        raise NotImplementedError("Only `caller=\"torch\"` is supported.")

    def wrapper(function):
        annotations = inspect.get_annotations(function) if hasattr(inspect, "get_annotations") else function.__annotations__
        parameters = inspect.signature(function).parameters
        try:
            types = tuple(annotations[name] for name in parameters)
        except KeyError as error:
            raise TypeError(f"Parameter `{error.args[0]}` has no arranged tensor as its annotation.") from None
        return Kernel(function, types, kernel_name=kernel_name)

    if func is None:
        return wrapper
    return wrapper(func)


class Kernel:
    """A compute kernel bound to hand-written gfx950 code."""

    def __init__(self, application, types, kernel_name=None):
        self.application = application
        self.types = tuple(types)
        self.kernel_name = kernel_name if kernel_name is not None else getattr(application, "__name__", "kernel")
        self.kind, self.details, self.program = recognition.identify(application, self.types)
        self.parameters = list(inspect.signature(application).parameters)
        self.meta_symbols = recognition.unbound_meta_symbols(self.types)
        self._plans = {}
        self._scalar_flags = tuple((t.ndim == 0 and not isinstance(t.dtype, Tensor), bool(t.constexpr)) for t in self.types)
        self._source_path = None
        self.last_plan = None  # description of the launch used by the latest call

    # `_source` mirrors the reference handle's attribute (src/ninetoothed/jit.py:121-125):
    # a path to a readable description of what runs
    @property
    def _source(self):
        if self._source_path is None:
            text = (
                f"# kernel `{self.kernel_name}`: recognised as `{self.kind}` {self.details}\n"
                f"# executed by libnt_hip.so ({runtime.LIBRARY_PATH})\n"
                f"# dataflow graph of the application (digest {self.program.digest}):\n" + self.program.describe() + "\n"
            )
            for program in getattr(self, "_map_programs", ()):
                import ctypes

                buffer = ctypes.create_string_buffer(1 << 16)
                if runtime.library().nt_map_source(ctypes.addressof(program), buffer, len(buffer)) == 0:
                    text += "# HIP source of the latest prepared launch:\n" + buffer.value.decode() + "\n"
            CACHE_DIR.mkdir(parents=True, exist_ok=True)
            path = CACHE_DIR / (hashlib.sha256(text.encode()).hexdigest() + ".txt")
            if not path.exists():
                path.write_text(text)
            self._source_path = str(path)
        return self._source_path

    # the reference's handle also carries `_kernel` (the compiled kernel) and `_launch`
    # (the launch function `__call__` forwards to), src/ninetoothed/jit.py:121-128
    @property
    def _kernel(self):
        return self

    def _launch(self, *args, **kwargs):
        return self(*args, **kwargs)

    def __call__(self, *args, **kwargs):
        if len(args) != len(self.types):
            raise TypeError(f"`{self.kernel_name}` takes {len(self.types)} positional arguments but {len(args)} were given.")
        key = self._signature(args, kwargs)
        plan = self._plans.get(key)
        if plan is None:
            plan = self._plans[key] = self._prepare(args, kwargs)
        self.last_plan = plan.description
        plan(args)

    # ---- plan construction ----------------------------------------------
    def _signature(self, args, kwargs):
        # on the path of every call: torch.Size, the stride tuple, dtype and device are hashable as they are
        parts = []
        for arg, (is_scalar, constexpr) in zip(args, self._scalar_flags):
            if is_scalar:
                parts.append((type(arg), arg if constexpr else None))
            elif getattr(arg, "is_nested", False):
                parts.append(_jagged_layout(arg) + (arg.dtype, arg.device))
            else:
                try:
                    parts.append((arg.shape, arg.stride(), arg.dtype, arg.device))
                except AttributeError:  # not a tensor: `_environment` says so
                    parts.append((type(arg), None))
        return tuple(parts), (tuple(sorted(kwargs.items())) if kwargs else ())

    def _environment(self, args, kwargs, check_device=True):
        import torch

        env = {}
        for name, arg, tensor in zip(self.parameters, args, self.types):
            source = tensor.source
            if tensor.ndim == 0 and not isinstance(tensor.dtype, Tensor):
                if isinstance(arg, torch.Tensor):
                    raise TypeError(f"`{name}` is a zero-dimensional tensor: pass a Python number.")
                continue
            if not isinstance(arg, torch.Tensor):
                raise TypeError(f"`{name}` must be a torch tensor, not `{type(arg).__name__}`.")
            if check_device and not arg.is_cuda:
                raise RuntimeError(f"`{name}` lives on `{arg.device}`; this build only runs on the GPU (there is no CPU path).")
            if arg.ndim != source.ndim:
                raise ValueError(f"`{name}` must have {source.ndim} dimensions, got {arg.ndim}.")
            if (source.jagged_dim is not None) != bool(getattr(arg, "is_nested", False)):
                raise TypeError(f"`{name}` is {'declared jagged: pass a `torch.jagged` nested tensor' if source.jagged_dim is not None else 'not declared jagged: pass a dense tensor'}.")
            if source.jagged_dim is not None:
                # sizes as the launch sees them (src/ninetoothed/tensor.py:621-637, generation.py:686-704):
                # the longest sequence along the jagged dimension, no stride along the batch
                if self.kind != "map":
                    raise UnsupportedProgram("Jagged tensors are only supported by the element-wise executor.")
                if arg._ragged_idx != source.jagged_dim:
                    raise ValueError(f"`{name}` is jagged along dimension {arg._ragged_idx}, declared along {source.jagged_dim}.")
                shape, strides = _jagged_layout(arg)
                for dim in range(source.ndim):
                    declared = source.shape[dim]
                    if isinstance(declared, Symbol) and declared.is_name:
                        env[declared.name] = shape[dim]
                    env[source.size_string(dim)] = shape[dim]
                    env[source.stride_string(dim)] = strides[dim]
                continue
            for dim in range(source.ndim):
                declared = source.shape[dim]
                if not isinstance(declared, Symbol) and int(declared) != arg.shape[dim]:
                    raise ValueError(f"Dimension {dim} of `{name}` was declared as {declared}, got {arg.shape[dim]}.")
                if isinstance(declared, Symbol) and declared.is_name:
                    env[declared.name] = arg.shape[dim]
                env[source.size_string(dim)] = arg.shape[dim]
                env[source.stride_string(dim)] = arg.stride(dim)
        for name, value in kwargs.items():
            env[name] = value
        for name in self.meta_symbols:
            env.setdefault(name, 1)  # index maps do not depend on block sizes; analyse with unit blocks
        return env

    def _prepare(self, args, kwargs):
        env = self._environment(args, kwargs)
        try:
            builder = getattr(self, "_prepare_" + self.kind)
            return builder(args, env)
        except KeyError as error:
            raise TypeError(f"`{self.kernel_name}` needs a value for {error.args[0]}; pass it by keyword.") from None

    def _tensor_dtype(self, *tensors, allowed):
        tags = {_dtype_tag(tensor.dtype) for tensor in tensors}
        if len(tags) != 1:
            raise UnsupportedProgram(f"Operands have different element types: {sorted(tags)}.")
        (tag,) = tags
        if tag not in allowed:
            raise UnsupportedProgram(f"No `{self.kind}` kernel for element type `{tag}` (supported: {', '.join(allowed)}).")
        return tag

    def _prepare_matmul(self, args, env):
        lhs, rhs, out = args
        kind, info = recognition.analyze_gemm(self.types[0], self.types[1], self.types[2], env)
        if kind == "empty":
            return _Plan("empty launch", lambda call_args: None)
        tag = self._tensor_dtype(lhs, rhs, allowed=("fp16", "bf16", "fp32", "fp8e5m2"))
        out_tag = _dtype_tag(out.dtype)
        cast = self.details.get("cast")
        if tag == "fp8e5m2":  # the second case of the reference's tests/test_matmul.py:61-88
            if kind in ("conv2d", "batched") or out_tag not in ("fp16", "fp32") or cast not in (None, out_tag):
                raise UnsupportedProgram("fp8 operands are supported for plain matmul into fp16 / fp32 only.")
            return self._gemm_plan(info, tag, out_tag, positions=(None, 0, 1, None, None, 2))
        if kind == "conv2d":
            if out_tag != tag or cast not in (None, tag):
                raise UnsupportedProgram("conv2d needs input, filter and output of one element type.")
            return self._conv2d_plan(info, tag, args)
        if cast is not None and cast != out_tag:
            raise UnsupportedProgram(f"The application rounds to `{cast}` but the output tensor holds `{out_tag}`.")
        if out_tag not in (tag, "fp32"):
            raise UnsupportedProgram(f"No matmul kernel writing `{out_tag}` from `{tag}` operands.")
        if kind == "batched":
            return self._batched_gemm_plan(info, tag, out_tag)
        return self._gemm_plan(info, tag, out_tag, positions=(None, 0, 1, None, None, 2))

    def _batched_gemm_plan(self, info, tag, out_tag):
        """One launch for all products of a batch (``launch_nt_batched_matmul``)."""
        lib = runtime.library()
        itemsize = 4 if tag == "fp32" else 2
        out_itemsize = 4 if out_tag == "fp32" else 2
        batch, m, n, k = info["batch"], info["m"], info["n"], info["k"]
        blocks = [info["blocks"][axis] if info["blocks"][axis] > 1 else 0 for axis in ("m", "n", "k")]
        dtype, out_dtype = runtime.DATA_TYPE_INDEX[tag], runtime.DATA_TYPE_INDEX[out_tag]

        def layout(matrix, rows, cols, shared_allowed):
            # (a dimension of one element has no coefficient in the index map: give it the stride of a dense matrix)
            col_stride = matrix.col_stride if cols > 1 or matrix.col_stride else 1
            row_stride = matrix.row_stride if rows > 1 or matrix.row_stride else (cols if col_stride == 1 else 1)
            shared = shared_allowed and batch > 1 and matrix.batch_stride == 0  # one matrix for every product
            return runtime.ArgumentTensor.from_layout(0, (1 if shared else batch, rows, cols), (matrix.batch_stride, row_stride, col_stride))

        a, b, c = info["a"], info["b"], info["c"]
        a_arg, b_arg, c_arg = layout(a, m, k, True), layout(b, k, n, True), layout(c, m, n, False)

        def launch(call_args):
            a_arg.data = call_args[0].data_ptr() + a.base * itemsize
            b_arg.data = call_args[1].data_ptr() + b.base * itemsize
            c_arg.data = call_args[2].data_ptr() + c.base * out_itemsize
            runtime.check(lib.launch_nt_batched_matmul(runtime.current_stream(), a_arg, b_arg, c_arg, dtype, out_dtype, *blocks))

        return _Plan(f"launch_nt_batched_matmul {batch}x{m}x{n}x{k} {tag}->{out_tag} blocks {blocks}", launch)

    def _prepare_addmm(self, args, env):
        input, mat1, mat2, beta, alpha, out = args
        kind, info = recognition.analyze_gemm(self.types[1], self.types[2], self.types[5], env, input_type=self.types[0])
        if kind == "empty":
            return _Plan("empty launch", lambda call_args: None)
        if _dtype_tag(mat1.dtype) == "fp8e5m2":  # the second case of the reference's tests/test_addmm.py:57-90
            tag = self._tensor_dtype(input, mat1, mat2, allowed=("fp8e5m2",))
            if self.details.get("cast") != "fp16" or _dtype_tag(out.dtype) != "fp16":
                raise UnsupportedProgram("addmm on fp8 operands rounds the product to fp16 and writes an fp16 tensor.")
            return self._gemm_plan(info, tag, "fp16", positions=(0, 1, 2, 3, 4, 5))
        tag = self._tensor_dtype(input, mat1, mat2, out, allowed=("fp16", "bf16", "fp32"))
        if self.details.get("cast") not in ((tag, None) if tag == "fp32" else (tag,)):
            raise UnsupportedProgram(f"The application rounds the product to `{self.details.get('cast')}` but the tensors hold `{tag}`.")
        return self._gemm_plan(info, tag, tag, positions=(0, 1, 2, 3, 4, 5))

    def _gemm_plan(self, info, tag, out_tag, positions):
        lib = runtime.library()
        itemsize = {"fp8e5m2": 1, "fp32": 4}.get(tag, 2)
        out_itemsize = 4 if out_tag == "fp32" else 2
        a, b, c, i = info["a"], info["b"], info["c"], info["input"]
        m, n, k = info["m"], info["n"], info["k"]
        blocks = [info["blocks"][axis] if info["blocks"][axis] > 1 else 0 for axis in ("m", "n", "k")]
        dtype, out_dtype = runtime.DATA_TYPE_INDEX[tag], runtime.DATA_TYPE_INDEX[out_tag]
        in_pos, a_pos, b_pos, beta_pos, alpha_pos, c_pos = positions

        def layout(matrix, rows, cols):
            # a dimension of one element has no coefficient in the index map (stride 0): give it the
            # stride of a dense matrix, so that a single row or column stays on the fast kernels
            col_stride = matrix.col_stride if cols > 1 or matrix.col_stride else 1
            row_stride = matrix.row_stride if rows > 1 or matrix.row_stride else (cols if col_stride == 1 else 1)
            return (rows, cols), (row_stride, col_stride)

        a_arg = runtime.ArgumentTensor.from_layout(0, *layout(a, m, k))
        b_arg = runtime.ArgumentTensor.from_layout(0, *layout(b, k, n))
        c_arg = runtime.ArgumentTensor.from_layout(0, *layout(c, m, n))
        # block sizes left to the tuner (all meta): like the reference's autotuned kernels, the
        # first launch of a new problem times the candidates once (src/ninetoothed/generation.py:372-516)
        from ninetoothed_amd import auto_tuner

        state = {"tune": blocks == [0, 0, 0] and min(m, n, k) > 0 and auto_tuner.enabled()}
        if state["tune"]:
            auto_tuner.load_once()
            rhs_layout = 0 if b_arg.strides[1] == 1 else (1 if b_arg.strides[0] == 1 else 2)
            state["tune"] = auto_tuner.lookup(dtype, out_dtype, m, n, k, i is not None, rhs_layout) < 0

        def maybe_tune(call_args, input_arg, beta, alpha):
            state["tune"] = False
            out = call_args[c_pos]
            sources = [call_args[p] for p in (in_pos, a_pos, b_pos) if p is not None]
            # timing launches rewrite the output; skip when it overlaps an operand
            if any(t.untyped_storage().data_ptr() == out.untyped_storage().data_ptr() for t in sources):
                return
            instance, _ = auto_tuner.tune(input_arg, a_arg, b_arg, beta, alpha, c_arg, dtype, out_dtype)
            # inside a graph capture nothing is timed (-1): the next call outside one tunes; -2: nothing to choose from
            state["tune"] = instance == -1

        if i is not None:
            i_arg = runtime.ArgumentTensor.from_layout(0, (m, n), (i.row_stride, i.col_stride))  # (a stride of 0 is a broadcast here)

            def launch(call_args):
                a_arg.data = call_args[a_pos].data_ptr() + a.base * itemsize
                b_arg.data = call_args[b_pos].data_ptr() + b.base * itemsize
                c_arg.data = call_args[c_pos].data_ptr() + c.base * out_itemsize
                i_arg.data = call_args[in_pos].data_ptr() + i.base * itemsize
                beta = runtime.ArgumentTensor.from_scalar(float(call_args[beta_pos]))
                alpha = runtime.ArgumentTensor.from_scalar(float(call_args[alpha_pos]))
                if state["tune"]:
                    maybe_tune(call_args, i_arg, beta, alpha)
                runtime.check(lib.launch_nt_addmm(runtime.current_stream(), i_arg, a_arg, b_arg, beta, alpha, c_arg, dtype, *blocks))

            return _Plan(f"launch_nt_addmm {m}x{n}x{k} {tag} blocks {blocks}", launch)

        def launch(call_args):
            a_arg.data = call_args[a_pos].data_ptr() + a.base * itemsize
            b_arg.data = call_args[b_pos].data_ptr() + b.base * itemsize
            c_arg.data = call_args[c_pos].data_ptr() + c.base * out_itemsize
            if state["tune"]:
                null = runtime.ArgumentTensor.null()
                maybe_tune(call_args, null, null, null)
            runtime.check(lib.launch_nt_matmul(runtime.current_stream(), a_arg, b_arg, c_arg, dtype, out_dtype, *blocks))

        return _Plan(f"launch_nt_matmul {m}x{n}x{k} {tag}->{out_tag} blocks {blocks}", launch)

    def _conv2d_plan(self, info, tag, args):
        lib = runtime.library()
        dtype = runtime.DATA_TYPE_INDEX[tag]
        pad_h, pad_w = info["pad_h"], info["pad_w"]
        blocks = [info["blocks"][axis] if info["blocks"][axis] > 1 else 0 for axis in ("m", "n", "k")]
        steps = (info.get("stride_h", 1), info.get("stride_w", 1), info.get("dilation_h", 1), info.get("dilation_w", 1))
        if steps != (1, 1, 1, 1) or not info.get("fits", True):
            # windows that move by more than one position, taps that lie apart, or one window hanging over the edge

            x, w, y = (runtime.ArgumentTensor.like(tensor) for tensor in args)  # (a plan serves one layout: only the addresses change)

            def launch_strided(call_args):
                x.data, w.data, y.data = call_args[0].data_ptr(), call_args[1].data_ptr(), call_args[2].data_ptr()
                runtime.check(lib.launch_nt_conv2d_strided(runtime.current_stream(), x, w, y, dtype, pad_h, pad_w, *steps, *blocks))

            return _Plan(
                f"launch_nt_conv2d_strided gemm {info['m']}x{info['n']}x{info['k']} {tag} padding ({pad_h}, {pad_w}) stride {steps[:2]} dilation {steps[2:]}", launch_strided
            )

        from ninetoothed_amd import auto_tuner

        # block sizes left to the tuner: the first launch of a new problem times the ways to run it
        state = {"tune": blocks == [0, 0, 0] and auto_tuner.enabled()}
        if state["tune"]:
            auto_tuner.load_once()

        x, w, y = (runtime.ArgumentTensor.like(tensor) for tensor in args)  # (a plan serves one layout: only the addresses change)

        def launch(call_args):
            x.data, w.data, y.data = call_args[0].data_ptr(), call_args[1].data_ptr(), call_args[2].data_ptr()
            if state["tune"]:
                state["tune"] = False
                out = call_args[2]
                if all(t.untyped_storage().data_ptr() != out.untyped_storage().data_ptr() for t in call_args[:2]):
                    # (timing launches rewrite the output; inside a graph capture nothing is timed: try again later)
                    state["tune"] = auto_tuner.tune_conv2d(x, w, y, dtype, pad_h, pad_w) == -1
            runtime.check(lib.launch_nt_conv2d(runtime.current_stream(), x, w, y, dtype, pad_h, pad_w, *blocks))

        return _Plan(f"launch_nt_conv2d gemm {info['m']}x{info['n']}x{info['k']} {tag} padding ({pad_h}, {pad_w})", launch)

    def _prepare_softmax(self, args, env):
        kind, info = recognition.analyze_softmax(self.types[0], self.types[1], env)
        if kind == "empty":
            return _Plan("empty launch", lambda call_args: None)
        tag = self._tensor_dtype(*args, allowed=("fp32", "fp16", "bf16"))
        lib = runtime.library()
        dtype = runtime.DATA_TYPE_INDEX[tag]
        block = info["input"]["block"]

        input, output = (runtime.ArgumentTensor.like(tensor) for tensor in args[:2])  # (a plan serves one layout: only the addresses change)

        def launch(call_args):
            input.data, output.data = call_args[0].data_ptr(), call_args[1].data_ptr()
            runtime.check(lib.launch_nt_softmax(runtime.current_stream(), input, output, dtype, block))

        return _Plan(f"launch_nt_softmax {info['input']['rows']}x{info['input']['cols']} {tag} block {block}", launch)

    def _prepare_map(self, args, env):
        """Element-wise / reducing programs: one interpreter launch per store."""
        import ctypes

        from ninetoothed_amd import mapping

        lib = runtime.library()
        tensor_params = [p for p, t in enumerate(self.types) if not (t.ndim == 0 and not isinstance(t.dtype, Tensor))]
        for p in tensor_params:
            if args[p].numel() > 0 and _storage(args, p).data_ptr() % args[p].element_size():
                raise UnsupportedProgram("Tensor data must be aligned to its element size.")
        launches = []
        for store in self.program.stores:
            built = mapping.build(store, self.types, args, env, lambda p: _dtype_tag(_storage(args, p).dtype), lambda p: _storage(args, p).data_ptr())
            if built is not None:
                launches.append(built)
        if not launches:
            return _Plan("empty launch", lambda call_args: None)

        def launch(call_args):
            stream = runtime.current_stream()
            for program, _, scalar_slots, operand_params in launches:
                for slot, param in enumerate(operand_params):
                    program.operands[slot].data = _storage(call_args, param).data_ptr()
                for index, param in scalar_slots:
                    program.value_constants[index] = float(call_args[param])
                runtime.check(lib.launch_nt_map(stream, ctypes.addressof(program)))

        self._map_programs = [program for program, _, _, _ in launches]
        return _Plan("launch_nt_map " + "; ".join(description for _, description, _, _ in launches), launch)

    def _prepare_gemm_epilogue(self, args, env):
        """A matmul accumulator followed by element-wise work (bias, activation, scaling, residual):
        the product goes to an fp32 scratch tensor laid out like the output (what the reference
        holds in the accumulator tile), then the rest runs as a tile map over it."""
        import ctypes

        import torch

        from ninetoothed_amd import mapping

        lib = runtime.library()
        details = self.details
        lhs_pos, rhs_pos, out_pos = details["lhs"], details["rhs"], details["output"]
        kind, info = recognition.analyze_gemm(self.types[lhs_pos], self.types[rhs_pos], self.types[out_pos], env)
        if kind == "empty":
            return _Plan("empty launch", lambda call_args: None)
        if kind != "strided":
            raise UnsupportedProgram("A product with an element-wise epilogue needs plain strided matrices.")
        tag = self._tensor_dtype(args[lhs_pos], args[rhs_pos], allowed=("fp16", "bf16", "fp32"))
        out = args[out_pos]
        if out.numel() and not (out.is_contiguous() or out.t().is_contiguous()):
            raise UnsupportedProgram("The output of a product with an epilogue must be a dense matrix.")
        scratch_pos = len(args)
        gemm = self._gemm_plan(info, tag, "fp32", positions=(None, lhs_pos, rhs_pos, None, None, scratch_pos))

        def with_scratch(call_args):
            target = call_args[out_pos]
            scratch = torch.empty_strided(target.shape, target.stride(), dtype=torch.float32, device=target.device)
            return tuple(call_args) + (scratch,)

        types = self.types + (self.types[out_pos],)
        sample = with_scratch(args)
        built = mapping.build(
            details["epilogue"].stores[0], types, sample, env, lambda p: _dtype_tag(_storage(sample, p).dtype), lambda p: _storage(sample, p).data_ptr()
        )
        if built is None:
            return _Plan("empty launch", lambda call_args: None)
        program, description, scalar_slots, operand_params = built

        def launch(call_args):
            extended = with_scratch(call_args)  # from torch's stream-ordered allocator: free again once both launches are queued
            gemm(extended)
            for slot, param in enumerate(operand_params):
                program.operands[slot].data = _storage(extended, param).data_ptr()
            for index, param in scalar_slots:
                program.value_constants[index] = float(extended[param])
            runtime.check(lib.launch_nt_map(runtime.current_stream(), ctypes.addressof(program)))

        self._map_programs = [program]
        return _Plan(f"{gemm.description}; launch_nt_map {description}", launch)

    def _prepare_attention(self, args, env):
        scaled = self.details["scale"]
        if scaled:
            q, k, v, is_causal, scale, o = args
            q_t, k_t, v_t, o_t = self.types[0], self.types[1], self.types[2], self.types[5]
        else:
            q, k, v, is_causal, o = args
            q_t, k_t, v_t, o_t = self.types[0], self.types[1], self.types[2], self.types[4]
        kind, info = recognition.analyze_attention(q_t, k_t, v_t, o_t, env)
        if kind == "empty":
            return _Plan("empty launch", lambda call_args: None)
        tag = self._tensor_dtype(q, k, v, o, allowed=("fp16", "bf16", "fp32"))
        lib = runtime.library()
        dtype = runtime.DATA_TYPE_INDEX[tag]
        o_pos = 5 if scaled else 4
        from ninetoothed_amd import auto_tuner

        # the first launch of a new problem times the loop variants (as the reference's autotuned kernel times its
        # block-size configurations, tests/test_attention.py:10-11 with src/ninetoothed/generation.py:372-516)
        state = {"tune": auto_tuner.enabled()}
        if state["tune"]:
            auto_tuner.load_once()

        positions = (0, 1, 2, o_pos)
        tensors = [runtime.ArgumentTensor.like(args[p]) for p in positions]  # (a plan serves one layout: only the addresses change)
        causal, causal_value = runtime.ArgumentTensor.scalar_slot(int)
        scale_arg, scale_value = runtime.ArgumentTensor.scalar_slot(float) if scaled else (runtime.ArgumentTensor.null(), None)

        def launch(call_args):
            for tensor, p in zip(tensors, positions):
                tensor.data = call_args[p].data_ptr()
            causal_value.value = int(bool(call_args[3]))
            if scaled:
                scale_value.value = float(call_args[4])
            if state["tune"]:
                state["tune"] = False
                out = call_args[o_pos]
                if all(call_args[p].untyped_storage().data_ptr() != out.untyped_storage().data_ptr() for p in (0, 1, 2)):
                    # (timing launches rewrite the output; inside a graph capture nothing is timed: try again later)
                    state["tune"] = auto_tuner.tune_attention(tensors[0], tensors[1], tensors[2], causal, scale_arg, tensors[3], dtype) == -1
            runtime.check(lib.launch_nt_attention(runtime.current_stream(), tensors[0], tensors[1], tensors[2], causal, scale_arg, tensors[3], dtype, 0, 0))

        return _Plan(f"launch_nt_attention q{info['q']['shape']} k{info['k']['shape']} {tag}", launch)


def _storage(args, param):
    """The dense tensor behind an operand of a tile map: the argument itself, the values of a
    jagged argument, or (``(position, "offsets")``) the sequence offsets of a jagged argument."""
    if isinstance(param, tuple):
        return args[param[0]].offsets()
    arg = args[param]
    return arg.values() if getattr(arg, "is_nested", False) else arg


def _jagged_layout(arg):
    """(shape, strides) a jagged nested tensor is launched with: batch entries of the longest
    length, laid over the values with no stride along the batch (the reference reads the
    longest length the same way at every call, src/ninetoothed/torchifier.py:33-36)."""
    values, offsets = arg.values(), arg.offsets()
    jagged_dim = arg._ragged_idx
    longest = int(offsets.diff().max().item()) if offsets.numel() > 1 else 0
    shape = [offsets.numel() - 1] + [longest if dim == jagged_dim else values.shape[dim - 1] for dim in range(1, arg.ndim)]
    strides = [0] + [values.stride(dim - 1) for dim in range(1, arg.ndim)]
    return tuple(shape), tuple(strides)


class _Plan:
    """A prepared launch.  Its argument structs are filled in per call, so calls from several
    host threads take turns (the launches themselves are asynchronous)."""

    __slots__ = ("description", "launch", "_lock")

    def __init__(self, description, launch):
        import threading

        self.description = description
        self.launch = launch
        self._lock = threading.Lock()

    def __call__(self, args):
        with self._lock:
            self.launch(args)
