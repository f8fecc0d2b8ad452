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
    """marks a device-buffer argument; the tensor itself travels to call(), which keeps it alive until the kernel is done"""
    return t if t is not None else NULL


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def call(name, *args):
    argv = [C.c_void_p(a.data_ptr()) if isinstance(a, torch.Tensor) else a for a in args]
    err = getattr(camx(), name)(*argv, stream())
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


def _row_scale(r):
    """max |r| over the last axis (the row or head an element belongs to), broadcast back"""
    r = np.abs(r)
    return np.maximum(r.max(axis=-1, keepdims=True) if r.ndim else r, 1e-30)


# Outputs behind the 128-point Hadamard transform of fp16-rounded values (the Q8 line's q16 and K rows): a one-ulp difference in one
# rotary output before the rounding moves that input by 2^-10 of its size at most, and every output of the head by 1 / sqrt(128) of
# that; by Parseval the largest output of a head is at least (largest input) / sqrt(128), so one such flip stays under 2^-10 of the
# head's largest output. Twice that as the floor.
HADAMARD_FLOOR = 2.0 ** -9


def close_fp32(a, ref, rel=1e-5, floor=None):
    """per element: |a - ref| <= rel * |ref| + floor * (max |ref| of the element's row), floor = rel / 10 unless given. The second term covers outputs that are a
    difference of products (a rotary pair, a gated sum), whose error scales with the operands and not with the result; it is tied to the
    element's own row, so a small value next to a large one in another row gets no slack from it."""
    a = np.asarray(a, np.float64); ref = np.asarray(ref, np.float64)
    return bool((np.abs(a - ref) <= rel * np.abs(ref) + (0.1 * rel if floor is None else floor) * _row_scale(ref)).all())


def close_16(bits, ref_bits, kind, rel=1e-5, floor=None):
    """16-bit outputs within one unit in the last place of the reference value, plus the fp32 bound above; kind 'f16' | 'bf16'"""
    bits = np.asarray(bits, np.uint16); ref_bits = np.asarray(ref_bits, np.uint16)
    if kind == 'f16':
        a = bits.view(np.float16).astype(np.float64); r = ref_bits.view(np.float16).astype(np.float64)
        ulp = np.abs(np.spacing(np.abs(ref_bits.view(np.float16)))).astype(np.float64)
    else:
        a = (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64); r = (ref_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        ulp = np.abs(r) * 2.0 ** -7 + 2.0 ** -133
    return bool((np.abs(a - r) <= ulp + rel * np.abs(r) + (0.1 * rel if floor is None else floor) * _row_scale(r)).all())
