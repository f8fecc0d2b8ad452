"""TEST INFRASTRUCTURE ONLY (like everything under oracle/): numpy decoders of the GGUF block formats whose embedding rows this library gathers on the device: Q4_K and Q8_0, in
float32 with every product and the difference rounded separately, so the device rows can be compared bit for bit.
Mirrors `q4_k`, `q8_0` and `dequant` of the reference's python/caminus/own_dequant.py:28-37, 202-206 (the other formats of
that module have no device kernel here).

  Q4_K  144 bytes / 256 values: d, dmin (fp16) | 12 bytes of 6-bit (scale, min) x 8 | 128 bytes of nibbles, 64 values per
        32-byte chunk: low nibbles first, then high.   y = (d * sc) * q - dmin * m
  Q8_0  34 bytes / 32 values: d (fp16) | 32 int8.     y = d * q
"""
import numpy as np

BLOCK = {'Q4_K': (256, 144), 'Q8_0': (32, 34)}     # values, bytes


def _half(b):
    return np.ascontiguousarray(b).view('<f2').astype(np.float32)


def _scales_mins(s):
    """12 packed bytes per block -> (sc [nb, 8], m [nb, 8]) as float32"""
    lo4, hi4, ext = s[:, 0:4], s[:, 4:8], s[:, 8:12]
    sc = np.concatenate([lo4 & 63, (ext & 0x0F) | ((lo4 >> 6) << 4)], axis=1)
    m = np.concatenate([hi4 & 63, (ext >> 4) | ((hi4 >> 6) << 4)], axis=1)
    return sc.astype(np.float32), m.astype(np.float32)


def q4_k(raw):
    b = np.asarray(raw, dtype=np.uint8).reshape(-1, 144)
    d, dmin = _half(b[:, 0:2]), _half(b[:, 2:4])                    # [nb, 1]
    sc, m = _scales_mins(b[:, 4:16])
    nib = b[:, 16:144].reshape(-1, 4, 32)
    q = np.stack([nib & 0x0F, nib >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)     # sub-block 2 n (+ 1 for the high nibbles)
    scale = (d * sc).astype(np.float32)[:, :, None]
    offs = (dmin * m).astype(np.float32)[:, :, None]
    return ((scale * q).astype(np.float32) - offs).astype(np.float32).reshape(-1)


def q8_0(raw):
    b = np.asarray(raw, dtype=np.uint8).reshape(-1, 34)
    return (_half(b[:, 0:2]) * b[:, 2:34].view(np.int8).astype(np.float32)).astype(np.float32).reshape(-1)


DECODERS = {'Q4_K': (256, 144, q4_k), 'Q8_0': (32, 34, q8_0)}


def dequant(raw, type_name, n_values):
    if type_name not in DECODERS:
        raise ValueError(f'own_dequant: {type_name} is not decoded here ({sorted(DECODERS)})')
    qk, bs, fn = DECODERS[type_name]
    if n_values % qk:
        raise ValueError(f'own_dequant: {n_values} values is not a whole number of {type_name} blocks ({qk})')
    raw = np.asarray(raw, dtype=np.uint8).reshape(-1)
    need = n_values // qk * bs
    if raw.size < need:
        raise ValueError(f'own_dequant: {raw.size} bytes < {need} for {n_values} {type_name} values')
    return fn(raw[:need])
