"""ctypes binding of libgq_hip.so, the HIP (gfx950) library behind the group-quantization path.

Stands where the reference imports its JIT-compiled pybind11 module
(popxl_addons/ops/group_quantize_decompress/group_quantize_decompress.py:4-6).  There is no
CPU fallback: a missing library or a non-zero return code raises.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_DEFAULT_LIB = os.path.join(os.path.dirname(_PKG_DIR), "lib", "libgq_hip.so")

GQ_ABI_VERSION = 1
GQ_ERR_NULL_POINTER = -1
GQ_ERR_BAD_SHAPE = -2
GQ_ERR_MISALIGNED = -3
GQ_ERR_UNSUPPORTED = -4
GQ_ERR_NO_DEVICE = -5

# every symbol declared in include/gq_hip.h
EXPORTS = (
    "gq_abi_version",
    "gq_last_error",
    "gq_set_option",
    "gq_decompress_f16",
    "gq_decompress_f16_transposed",
    "gq_gemv_f16",
    "gq_gemm_f16",
    "gq_linear_f16",
    "gq_compress_f16",
)


class GQHipError(RuntimeError):
    """A libgq_hip entry point returned a non-zero code."""

    def __init__(self, function, code, message):
        super().__init__(f"{function} failed with code {code}: {message}")
        self.function = function
        self.code = code


_lib = None


def library_path():
    return os.environ.get("GQ_HIP_LIBRARY", _DEFAULT_LIB)


def load():
    """Load the shared library once; raise if it is not built (python popxl-addons_amd/build.py)."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"libgq_hip.so not found at {path}: build it with `python popxl-addons_amd/build.py` "
            "(there is no CPU fallback for the device ops)"
        )
    lib = ctypes.CDLL(path)
    p, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.gq_abi_version.argtypes = []
    lib.gq_abi_version.restype = ctypes.c_int
    lib.gq_last_error.argtypes = []
    lib.gq_last_error.restype = ctypes.c_char_p
    lib.gq_set_option.argtypes = [ctypes.c_char_p, i64]
    lib.gq_set_option.restype = ctypes.c_int
    for name in ("gq_decompress_f16", "gq_decompress_f16_transposed"):
        fn = getattr(lib, name)
        fn.argtypes = [p, p, p, p, i64, i64, i64, p]
        fn.restype = ctypes.c_int
    for name in ("gq_gemv_f16", "gq_gemm_f16", "gq_linear_f16"):
        fn = getattr(lib, name)
        fn.argtypes = [p, i64, p, p, p, p, p, i64, i64, i64, p]
        fn.restype = ctypes.c_int
    lib.gq_compress_f16.argtypes = [p, p, p, p, p, i64, i64, i64, p]
    lib.gq_compress_f16.restype = ctypes.c_int
    if lib.gq_abi_version() != GQ_ABI_VERSION:
        raise ImportError(f"{path}: ABI version {lib.gq_abi_version()} != expected {GQ_ABI_VERSION}")
    _lib = lib
    return lib


def last_error():
    return load().gq_last_error().decode("utf-8", "replace")


def call(name, *args):
    """Call an entry point; raise GQHipError on a non-zero return."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise GQHipError(name, rc, lib.gq_last_error().decode("utf-8", "replace"))


def set_option(name, value):
    call("gq_set_option", name.encode(), int(value))
