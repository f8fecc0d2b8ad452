"""ctypes binding of libcamx.so's C ABI (include/camx.h). One process-wide handle; every entry point returns an int
(0 or a hipError_t). There is no CPU or PyTorch fallback: loading fails loudly when the library is absent."""
import ctypes
import os

from . import kernels as _kernels

_lib = None


def load():
    global _lib
    if _lib is None:
        d, where = _kernels.kernel_dir()
        p = os.path.join(d, _kernels.LIBNAME)
        if not os.path.isfile(p):
            raise FileNotFoundError(_kernels.missing_message('camx', d, where))
        # one HIP runtime per process: PyTorch ships its own libamdhip64.so, and the library must resolve to the copy that owns the
        # caller's device pointers. With torch loaded first the dynamic loader hands the library that copy; the other way round the
        # library binds to the system's runtime and refuses torch's pointers (hipErrorInvalidValue).
        import torch  # noqa: F401
        _lib = ctypes.CDLL(p)
        _lib.camx_error_string.restype = ctypes.c_char_p
        _lib.camx_error_string.argtypes = [ctypes.c_int]
    return _lib


def check(err):
    if err != 0:
        raise RuntimeError(f'HIP error {err}: {load().camx_error_string(int(err)).decode()}')
