"""Helpers of the GPU parity tests: device buffers through torch (allocation only), calls through the C ABI."""
import ctypes as C

import numpy as np
import torch

from caminus_amd.device import lib as _lib

DEV = 'cuda:0'
I, F, L64 = C.c_int, C.c_float, C.c_int64
NULL = C.c_void_p(None)


def camx():
    return _lib.load()


def dev(a):
    """numpy array -> device tensor holding the same bytes (uint16 carried as int16)"""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16: return torch.from_numpy(a.view(np.int16)).to(DEV)
    if a.dtype == np.uint32: return torch.from_numpy(a.view(np.int32)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def host(t, dtype=None):
    a = t.detach().cpu().numpy()
    return a.view(dtype) if dtype is not None else a


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else NULL


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def call(name, *args):
    err = getattr(camx(), name)(*args, stream())
    _lib.check(err)
    torch.cuda.synchronize()


def bits_equal(a, b):
    a = np.ascontiguousarray(a); b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype.itemsize == b.dtype.itemsize and np.array_equal(a.view(np.uint8), b.view(np.uint8))


def outliers(rng, shape, frac=1e-3, scale=50.0):
    """N(0, 1) activations with `frac` of the entries scaled by `scale`"""
    x = rng.standard_normal(shape).astype(np.float32)
    m = rng.random(shape) < frac
    x[m] *= np.float32(scale)
    return x
