"""The position-span checks and KV row geometry the launch wrappers share. Mirrors the corresponding helpers of the
reference's python/caminus/engine/k3.py (ContextBoundsError :413-420, check_span :423-437, kv_pos_bytes :530-532,
kv_rows :535-540); the persistent tape engine of that module is not part of this library."""
import numpy as np

from ..errors import InvalidKVEncoding, NumericalFailure   # noqa: F401  (re-exported as in the reference module)

YARN_TABLE_FLOATS = 65      # freq[64] | mscale appended to the rotary parameter block in the long-context mode


class ContextBoundsError(IndexError):
    """a position (or a lazy-commit count) outside what the caller's buffers hold; raised on the host before any launch"""


def check_span(i0, n, max_ctx, commit=None, ntok=None, what='pass'):
    """positions i0 .. i0 + n - 1 must lie in [0, max_ctx); a commit count (when given) in [0, ntok]"""
    if isinstance(i0, bool) or not isinstance(i0, (int, np.integer)):
        raise ContextBoundsError(f'k3 {what}: position {i0!r} is not an int')
    i0, n = int(i0), int(n)
    if i0 < 0 or n < 1 or i0 + n > max_ctx:
        raise ContextBoundsError(f'k3 {what}: positions {i0} .. {i0 + n - 1} outside the KV cache [0, {max_ctx}) '
                                 f'(max_ctx {max_ctx}; build the engine with a larger max_ctx)')
    if commit is not None:
        if isinstance(commit, bool) or not isinstance(commit, (int, np.integer)) or not 0 <= int(commit) <= ntok:
            raise ContextBoundsError(f'k3 {what}: commit {commit!r} outside [0, {ntok}] (tokens of the previous pass)')


def kv_pos_bytes(M, q8):
    """bytes of one position's [K | V] row with M values each: Q8 blocks of 34 bytes per 32 values, or fp16"""
    return 2 * (M // 32) * 34 if q8 else 4 * M


def kv_rows(cache, M, q8):
    """positions a cache tensor holds, from its byte size"""
    pb = kv_pos_bytes(M, q8)
    nb = cache.numel() * cache.element_size()
    if q8 and M % 32:
        raise ValueError(f'k3 KV cache: {M} values per position is not a whole number of q8_0 blocks')
    if nb % pb or not 0 < nb // pb < 2 ** 31:
        raise ValueError(f'k3 KV cache: {nb} bytes is not a whole number of {pb}-byte positions')
    return nb // pb
