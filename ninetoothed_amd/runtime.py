"""ctypes binding of ``libnt_hip.so`` (the C ABI declared in
``include/ninetoothed_hip.h``).

Follows the calling convention of the reference's AOT loader
(src/ninetoothed/aot.py:704-751, 802-862): tensors are passed by value as
``{data, shape, strides}`` structs with element strides, Python scalars as
zero-dimensional tensors whose ``data`` points to a host ``double`` /
``int64``, the launch happens on the caller's current stream, and a non-zero
return value raises :class:`KernelLaunchError`.  There is no fallback: if the
library is missing, loading fails.
"""

import ctypes
import pathlib
import threading

LIBRARY_PATH = pathlib.Path(__file__).resolve().parent / "lib" / "libnt_hip.so"

NO_KERNEL = 1
# programs of the tuned-choice table (nt_tune_lookup, the cache file's problem lines)
TUNE_GEMM, TUNE_ATTENTION, TUNE_CONV2D = 0, 1, 2
SCRATCH_LIMIT = 2  # launch_nt_matmul_static_scratch: the call needs more than the fixed scratch array
STATIC_SCRATCH_BYTES = 16 << 20

# order of the reference's NineToothedDataType enum (src/ninetoothed/aot.py:524-537)
DATA_TYPES = ("i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "fp16", "bf16", "fp32", "fp64", "fp8e5m2")  # the last one extends the enum
DATA_TYPE_INDEX = {name: index for index, name in enumerate(DATA_TYPES)}


class KernelLaunchError(RuntimeError):
    def __init__(self, error_code):
        self.error_code = error_code
        super().__init__(f"Kernel launch failed with error code: {error_code}.")


class ArgumentTensor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("shape", ctypes.POINTER(ctypes.c_uint64)),
        ("strides", ctypes.POINTER(ctypes.c_int64)),
    ]

    @staticmethod
    def from_layout(data_ptr, shape, strides):
        shape_array = (ctypes.c_uint64 * max(len(shape), 1))(*shape)
        strides_array = (ctypes.c_int64 * max(len(strides), 1))(*strides)
        tensor = ArgumentTensor(data_ptr, shape_array, strides_array)
        tensor._keepalive = (shape_array, strides_array)
        return tensor

    @staticmethod
    def from_torch_tensor(tensor):
        argument = ArgumentTensor.from_layout(tensor.data_ptr(), tuple(tensor.shape), tuple(tensor.stride()))
        argument._torch_tensor = tensor
        return argument

    @staticmethod
    def like(tensor):
        """The layout of ``tensor`` without its address: a launch that serves one (shape, strides) signature keeps
        such an argument and only sets ``data`` per call."""
        return ArgumentTensor.from_layout(0, tuple(tensor.shape), tuple(tensor.stride()))

    @staticmethod
    def scalar_slot(kind):
        """A zero-dimensional tensor over a host buffer that stays (``float`` -> double, ``int`` -> int64); returns
        the argument and the buffer, whose ``value`` a launch sets per call."""
        buffer = ctypes.c_double(0.0) if kind is float else ctypes.c_int64(0)
        argument = ArgumentTensor(ctypes.addressof(buffer), None, None)
        argument._keepalive = buffer
        return argument, buffer

    @staticmethod
    def from_scalar(value):
        """A zero-dimensional tensor: host double for floats, host int64 otherwise."""
        buffer = ctypes.c_double(value) if isinstance(value, float) else ctypes.c_int64(int(value))
        argument = ArgumentTensor(ctypes.addressof(buffer), None, None)
        argument._keepalive = buffer
        return argument

    @staticmethod
    def null():
        return ArgumentTensor(None, None, None)


_T = ArgumentTensor
_I = ctypes.c_int
_S = ctypes.c_void_p

_SIGNATURES = {
    "launch_nt_matmul": (_S, _T, _T, _T, _I, _I, _I, _I, _I),
    "launch_nt_matmul_static_scratch": (_S, _T, _T, _T, _I, _I, _I, _I, _I),
    "launch_nt_batched_matmul": (_S, _T, _T, _T, _I, _I, _I, _I, _I),
    "launch_nt_addmm": (_S, _T, _T, _T, _T, _T, _T, _I, _I, _I, _I),
    "launch_nt_softmax": (_S, _T, _T, _I, _I),
    "launch_nt_softmax_config": (_S, _I, _T, _T, _I, _I),
    "launch_nt_attention": (_S, _T, _T, _T, _T, _T, _T, _I, _I, _I),
    "launch_nt_conv2d": (_S, _T, _T, _T, _I, _I, _I, _I, _I, _I),
    "launch_nt_conv2d_strided": (_S, _T, _T, _T, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I),
    "launch_nt_gemm_config": (_S, _I, _T, _T, _T, _T, _T, _T, _I, _I),
    "nt_tune_gemm": (_S, _T, _T, _T, _T, _T, _T, _I, _I, _I, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)),
    "nt_tune_attention": (_S, _T, _T, _T, _T, _T, _T, _I, _I, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)),
    "nt_tune_conv2d": (_S, _T, _T, _T, _I, _I, _I, _I, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)),
    "nt_tune_lookup": (_I, ctypes.POINTER(ctypes.c_int), _I),
    "nt_last_launch": (ctypes.c_char_p, _I),
    "launch_nt_map": (_S, ctypes.c_void_p),
    "nt_map_source": (ctypes.c_void_p, ctypes.c_char_p, _I),
    "nt_tune_cache_save": (ctypes.c_char_p,),
    "nt_tune_cache_load": (ctypes.c_char_p, ctypes.POINTER(ctypes.c_int)),
    "nt_tune_cache_lookup": (_I, _I, _I, _I, _I, _I),
    "nt_tune_file_format": (),
    "nt_gemm_num_configs": (),
    "nt_gemm_config_name": (_I, ctypes.c_char_p, _I),
}

_library = None
_lock = threading.Lock()


def library():
    """Loads ``libnt_hip.so`` once; raises if it has not been built."""
    global _library
    if _library is not None:
        return _library
    with _lock:
        if _library is None:
            if not LIBRARY_PATH.exists():
                raise RuntimeError(
                    f"{LIBRARY_PATH} is missing: build it with `python -m ninetoothed_amd.build_library` (needs hipcc). "
                    "There is no fallback path."
                )
            lib = ctypes.CDLL(str(LIBRARY_PATH))
            for name, argtypes in _SIGNATURES.items():
                function = getattr(lib, name)
                function.argtypes = list(argtypes)
                function.restype = ctypes.c_int
            lib.nt_version.restype = ctypes.c_char_p
            lib.nt_version.argtypes = []
            lib.nt_release_workspaces.restype = None
            lib.nt_release_workspaces.argtypes = []
            _library = lib
    return _library


def exported_symbols():
    return tuple(_SIGNATURES) + ("nt_version", "nt_release_workspaces")


def check(result):
    if result != 0:
        raise KernelLaunchError(result)


def current_stream():
    """The raw handle of torch's current stream on the current device (what the
    reference's launcher passes, src/ninetoothed/aot.py:834-856)."""
    import torch

    try:
        return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device()))
    except AttributeError:  # a torch without the private accessor
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def last_launch():
    """Which kernel served this thread's latest ``launch_nt_*`` call (instance, variant or path by index and
    description), as the library reports it."""
    buffer = ctypes.create_string_buffer(256)
    check(library().nt_last_launch(buffer, len(buffer)))
    return buffer.value.decode()


def gemm_config_names():
    lib = library()
    names = []
    for index in range(lib.nt_gemm_num_configs()):
        buffer = ctypes.create_string_buffer(160)
        check(lib.nt_gemm_config_name(index, buffer, len(buffer)))
        names.append(buffer.value.decode())
    return names
