"""Append fp32 K / V rows to a Q8 KV cache, unrotated: the host side of camx_own_kv_q8_append.

A cache row is [K blocks | V blocks]; a block is 34 bytes (little-endian fp16 scale, 32 int8 codes) for 32 consecutive
values. This file offers the reference launcher's class (python/caminus/device/kv_codec.py:34-101): Q8KVCodec(device,
module=None) with append(k, ldk, v, ldv, M, cache, pos0, T, err, rows=None) and check(err), raising the same exception
types in the same order: argument validation, position span, buffer checks, and only then the first GPU call.

Protocol. The caller zeroes the int32 word `err`, queues any number of appends, then calls check(err) before reading the
rows. Kernels only ever OR bits into the word: ERR_SPAN (a position outside the rows), ERR_NUMERICAL (a block the encoder
refuses: non-finite input, or a nonzero block whose scale or reciprocal leaves the finite nonzero range), ERR_LAYOUT
(M or a stride the kernel cannot serve). A refused block keeps whatever bytes it had while its neighbours are written, so
one bit spoils the whole append.
"""
import ctypes
from numbers import Integral

import torch

from .bufcheck import LaunchCheck
from .hip import Module

INT_MAX = 2 ** 31 - 1
ERR_SPAN, ERR_NUMERICAL, ERR_LAYOUT = 1, 2, 4
_ERR_NAMES = {ERR_SPAN: 'span', ERR_NUMERICAL: 'numerical domain', ERR_LAYOUT: 'layout'}
_BLOCK_VALUES, _BLOCK_BYTES = 32, 34

_check = LaunchCheck('kv_codec', align=4)


def _integer(value, name, minimum=0):
    """a C int in [minimum, INT_MAX]; bools and floats are refused"""
    if isinstance(value, Integral) and not isinstance(value, bool) and minimum <= value <= INT_MAX:
        return int(value)
    raise ValueError(f'kv_codec: {name} must be an integer in [{minimum}, {INT_MAX}]')


def _explicit_cuda_device(device):
    if isinstance(device, (str, torch.device)):
        dev = torch.device(device)
        if dev.type == 'cuda' and dev.index is not None:
            return dev
    raise ValueError('kv_codec: device must be an explicitly indexed CUDA device')


def _cache_rows(cache, row_bytes, rows):
    """how many rows may be written: the whole view, or the caller's smaller `rows`"""
    if not (isinstance(cache, torch.Tensor) and cache.dtype == torch.uint8 and cache.numel() % row_bytes == 0):
        raise ValueError(f'kv_codec: cache must be uint8 whole rows of {row_bytes} bytes')
    held = _integer(cache.numel() // row_bytes, 'physical rows', 1)
    if rows is None:
        return held
    rows = _integer(rows, 'rows', 1)
    if rows > held:
        raise ValueError(f'kv_codec: rows {rows} exceed the cache view of {held} physical rows')
    return rows


class Q8KVCodec:
    """The codec on one device. Building it touches no GPU; the library is loaded by the first append that passed every
    host check. `module` injects a stand-in with an own_kv_q8_append attribute (a launch recorder in CPU tests)."""

    def __init__(self, device, module=None):
        self.dev = _explicit_cuda_device(device)
        self.module = module
        self.reader = module             # read() binds the library's own entry point lazily (a recorder serves both)

    def append(self, k, ldk, v, ldv, M, cache, pos0, T, err, rows=None):
        """Queue the encode of rows pos0 .. pos0 + T - 1 from k[t * ldk : t * ldk + M] and v[t * ldv : t * ldv + M].

        k, v: fp32 on this device, contiguous, large enough for the last row (they may alias each other). cache: uint8,
        a whole number of rows of 2 * (M / 32) * 34 bytes; `rows` narrows the writable prefix. err: int32, first word
        used. cache and err must overlap no other operand."""
        M = _integer(M, 'M', _BLOCK_VALUES)
        if M % _BLOCK_VALUES:
            raise ValueError('kv_codec: M must be divisible by 32')
        T = _integer(T, 'T', 1)
        ldk, ldv = _integer(ldk, 'ldk', M), _integer(ldv, 'ldv', M)
        pos0 = _integer(pos0, 'pos0')
        row_bytes = 2 * (M // _BLOCK_VALUES) * _BLOCK_BYTES
        rows = _cache_rows(cache, row_bytes, rows)

        from ..engine.k3 import check_span
        check_span(pos0, T, rows, what='own Q8 KV append')

        operands = {
            'k': (k, torch.float32, (T - 1) * ldk + M),
            'v': (v, torch.float32, (T - 1) * ldv + M),
            'cache': (cache, torch.uint8, rows * row_bytes, 2),
            'err': (err, torch.int32, 1),
        }
        _check(self.dev, 'own_kv_q8_append', operands, ('cache', 'err'))

        c_int = ctypes.c_int
        with torch.cuda.device(self.dev):
            if self.module is None:
                self.module = Module('kv_codec')
            self.module.own_kv_q8_append((T,), (256,), k, c_int(ldk), v, c_int(ldv), c_int(M), cache, c_int(pos0), c_int(rows), err)

    def read(self, cache, M, k, ldk, v, ldv, pos0, T, err, rows=None, row_ids=None):
        """Queue the decode of rows pos0 .. pos0 + T - 1 (or rows row_ids[0 .. T - 1], int32 on this device) into k / v: fp32, or
        fp16 (rounded from the fp32 value) when k is float16. The reference launcher has no decoder (its attention kernels
        decode blocks in place); the checks and the error word follow append()."""
        M = _integer(M, 'M', _BLOCK_VALUES)
        if M % _BLOCK_VALUES:
            raise ValueError('kv_codec: M must be divisible by 32')
        T = _integer(T, 'T', 1)
        ldk, ldv = _integer(ldk, 'ldk', M), _integer(ldv, 'ldv', M)
        pos0 = _integer(pos0, 'pos0')
        row_bytes = 2 * (M // _BLOCK_VALUES) * _BLOCK_BYTES
        rows = _cache_rows(cache, row_bytes, rows)
        if row_ids is None:
            from ..engine.k3 import check_span
            check_span(pos0, T, rows, what='own Q8 KV read')
        if not isinstance(k, torch.Tensor) or k.dtype not in (torch.float32, torch.float16):
            raise ValueError('kv_codec: k must be float32 or float16')
        if k.dtype == torch.float16 and (ldk % 4 or ldv % 4):
            raise ValueError('kv_codec: float16 rows need strides that are multiples of 4 (the rows are written 8 bytes at a time)')
        operands = {
            'cache': (cache, torch.uint8, rows * row_bytes, 2),
            'k': (k, k.dtype, (T - 1) * ldk + M, 8 if k.dtype == torch.float16 else 4),
            'v': (v, k.dtype, (T - 1) * ldv + M, 8 if k.dtype == torch.float16 else 4),
            'err': (err, torch.int32, 1),
        }
        if row_ids is not None:
            operands['row_ids'] = (row_ids, torch.int32, T)
        _check(self.dev, 'own_kv_q8_read', operands, ('k', 'v', 'err'))
        c_int = ctypes.c_int
        with torch.cuda.device(self.dev):
            if self.reader is None:
                self.reader = Module('camx')
            self.reader.camx_own_kv_q8_read((T,), (256,), cache, row_ids if row_ids is not None else ctypes.c_void_p(None), c_int(pos0), c_int(rows),
                                            c_int(M), k, c_int(ldk), v, c_int(ldv), err, c_int(T), c_int(int(k.dtype == torch.float16)))

    def check(self, err):
        """Synchronize the device, read the word, raise RuntimeError if any bit is set. The word is left as it is."""
        _check(self.dev, 'own_kv_q8_check', {'err': (err, torch.int32, 1)}, ())
        torch.cuda.synchronize(self.dev)
        word = int(err.view(-1)[0].item())
        if word == 0:
            return
        reasons = [name for bit, name in _ERR_NAMES.items() if word & bit]
        if word & ~sum(_ERR_NAMES):
            reasons.append('unknown error bits')
        raise RuntimeError(f'kv_codec: whole append result is unusable (err {word:#x}: {", ".join(reasons)})')
