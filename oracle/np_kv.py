"""TEST INFRASTRUCTURE ONLY (like everything under oracle/): numpy restatement of the Q8 KV row bytes and of the 128-point
Hadamard rotation that follows the reference's python/caminus/ref_kv.py:44-144 function by function (Q8KVLayout, hadamard128,
encode_q8_kv, decode_q8_kv: the same arguments, refusals and messages). It shares no code with oracle/camx_oracle.c, so the tests
compare the two bit for bit; as a pin it adds only that cross-check to the literal vectors.

A row is K then V, each the head-major vector cut into 32-value blocks of a little-endian fp16 scale and 32 signed bytes.
Encode: fp32 amax / 127, its fp32 reciprocal, fp32 product, round half away from zero; only the STORED scale is rounded to
half. A nonzero block needs a finite nonzero fp32 scale and reciprocal and a finite half scale; everything else is refused.
"""
from dataclasses import dataclass
from operator import index

import numpy as np

HADAMARD128_SCALE = np.float32(float.fromhex('0x1.6a09e6p-4'))        # float32(1 / sqrt(128))


def _count(value, name):
    err = ValueError(f'{name} must be a nonnegative integer')
    if isinstance(value, (bool, np.bool_)):
        raise err
    try:
        value = index(value)
    except TypeError:
        raise err from None
    if value < 0:
        raise err
    return value


@dataclass(frozen=True)
class Q8KVLayout:
    """[K blocks of all heads | V blocks of all heads], no padding"""
    kv_heads: int
    head_dim: int

    def __post_init__(self):
        heads, dim = _count(self.kv_heads, 'kv_heads'), _count(self.head_dim, 'head_dim')
        if not heads or not dim or dim % 32:
            raise ValueError('positive heads and head_dim divisible by 32 required')
        object.__setattr__(self, 'kv_heads', heads)
        object.__setattr__(self, 'head_dim', dim)

    @property
    def values(self):
        return self.kv_heads * self.head_dim

    @property
    def row_bytes(self):
        return 2 * (self.values // 32) * 34

    def cache_bytes(self, rows):
        return _count(rows, 'rows') * self.row_bytes


def hadamard128(x):
    """fp32 orthonormal Walsh-Hadamard transform of every 128-value head on the last axis, butterflies h = 1 .. 64 in order
    ((a, b) -> (a + b, a - b) for the pair (i, i + h), bit h of i clear), then one multiply by HADAMARD128_SCALE"""
    if not isinstance(x, np.ndarray) or x.dtype != np.float32:
        raise ValueError('hadamard128 needs a float32 numpy array')
    if x.ndim < 1 or x.shape[-1] != 128:
        raise ValueError('hadamard128: the last axis must be 128 values')
    y = x.reshape(-1, 128).copy()
    for h in (1, 2, 4, 8, 16, 32, 64):
        v = y.reshape(-1, 64 // h, 2, h)
        lo, hi = v[:, :, 0, :].copy(), v[:, :, 1, :].copy()
        v[:, :, 0, :], v[:, :, 1, :] = lo + hi, lo - hi
    return (y * HADAMARD128_SCALE).reshape(x.shape)


def _round_half_away(p):
    """roundf of already-rounded fp32 products (exact in float64)"""
    p64 = p.astype(np.float64)
    return np.copysign(np.floor(np.abs(p64) + 0.5), p64)


def encode_q8_kv(k, v, layout):
    """float32 [rows, kv_heads, head_dim] x 2 -> uint8 [rows, row_bytes]"""
    for name, a in (('K', k), ('V', v)):
        if not isinstance(a, np.ndarray) or a.dtype != np.float32:
            raise ValueError(f'{name} must be a float32 numpy array')
        if a.ndim != 3 or a.shape[1:] != (layout.kv_heads, layout.head_dim):
            raise ValueError(f'{name} shape must be [rows, kv_heads, head_dim]')
        if not np.isfinite(a).all():
            raise ValueError(f'{name} contains nonfinite values')
    if k.shape != v.shape:
        raise ValueError('K and V shapes must match')
    rows = k.shape[0]
    blocks = np.concatenate([k.reshape(rows, -1), v.reshape(rows, -1)], axis=1).reshape(-1, 32)
    amax = np.abs(blocks).max(axis=1) if blocks.size else np.zeros(0, np.float32)
    with np.errstate(all='ignore'):
        d = (amax / np.float32(127)).astype(np.float32)
        inv = np.where(d != 0, np.float32(1) / np.where(d != 0, d, np.float32(1)), np.float32(0)).astype(np.float32)
        stored = d.astype('<f2')
    bad = (amax != 0) & ((d == 0) | ~np.isfinite(d) | ~np.isfinite(inv) | ~np.isfinite(stored))
    if bad.any():
        raise ValueError('nonzero block scale is outside the reference encode domain')
    q = _round_half_away((blocks * inv[:, None]).astype(np.float32))
    if (np.abs(q) > 127).any():
        raise ValueError('quantized code outside [-127, 127]')
    out = np.empty((blocks.shape[0], 34), np.uint8)
    out[:, :2] = stored.view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.astype(np.int8).view(np.uint8)
    return out.reshape(rows, layout.row_bytes)


def decode_q8_kv(raw, layout):
    """uint8 [rows, row_bytes] -> (K, V) float32 [rows, kv_heads, head_dim]; any finite half scale and any code decode"""
    if not isinstance(raw, np.ndarray) or raw.dtype != np.uint8:
        raise ValueError('raw must be a uint8 numpy array')
    if raw.ndim != 2 or raw.shape[1] != layout.row_bytes:
        raise ValueError('raw shape must be [rows, row_bytes]')
    b = np.ascontiguousarray(raw).reshape(-1, 34)
    d = b[:, :2].copy().view('<f2').reshape(-1).astype(np.float32)
    if not np.isfinite(d).all():
        raise ValueError('nonfinite stored scale')
    vals = (b[:, 2:].view(np.int8).astype(np.float32) * d[:, None]).reshape(raw.shape[0], 2, layout.kv_heads, layout.head_dim)
    return vals[:, 0], vals[:, 1]
