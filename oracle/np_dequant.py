"""TEST INFRASTRUCTURE ONLY (like everything under oracle/): numpy decoders of the GGUF block formats whose embedding rows this
library gathers on the device: Q4_K, Q8_0, IQ4_NL, IQ4_XS and IQ2_S, in float32 with every product and the difference rounded
separately, so the device rows can be compared bit for bit. Mirrors `q4_k`, `q8_0`, `iq4_nl`, `iq4_xs`, `iq2_s` and `dequant`
of the reference's python/caminus/own_dequant.py:28-37, 128-137, 202-206 (the other formats of that module have no device
kernel here). Written block-wise from the formats' layouts; the C oracle states the same formats one value at a time.

  Q4_K  144 bytes / 256 values: d, dmin (fp16) | 12 bytes of 6-bit (scale, min) x 8 | 128 bytes of nibbles, 64 values per
        32-byte chunk: low nibbles first, then high.   y = (d * sc) * q - dmin * m
  Q8_0  34 bytes / 32 values: d (fp16) | 32 int8.     y = d * q
  IQ4_NL 18 bytes / 32 values: d (fp16) | 16 bytes of 4-bit indices (low nibbles = values 0-15, high = 16-31).  y = d * KV[index]
  IQ4_XS 136 bytes / 256 values: d (fp16) | scales_h (u16: 2 high bits per sub-block) | scales_l[4] (low 4 bits, two per
        byte) | 128 index bytes, 16 per sub-block of 32 as IQ4_NL.   y = (d * (scale6 - 32)) * KV[index]
  IQ2_S 82 bytes / 256 values: d (fp16) | qs[32] | signs[32] | qh[8] | scales[8]; 8 values per 10-bit codebook index
        qs | (2 bits of qh) << 8; a scale nibble per 16 values.   y = ((d * (0.5 + s)) * 0.25) * magnitude * (+-1)
"""
import numpy as np

BLOCK = {'Q4_K': (256, 144), 'Q8_0': (32, 34), 'IQ4_NL': (32, 18), 'IQ4_XS': (256, 136), 'IQ2_S': (256, 82)}     # values, bytes
KV_IQ4 = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


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


def _nibble_values(qs):
    """[..., 16] index bytes -> [..., 32] float32 values: the low nibbles, then the high ones"""
    return KV_IQ4[np.concatenate([qs & 0x0F, qs >> 4], axis=-1)]


def iq4_nl(raw):
    b = np.asarray(raw, dtype=np.uint8).reshape(-1, 18)
    return (_half(b[:, 0:2]) * _nibble_values(b[:, 2:18])).astype(np.float32).reshape(-1)


def iq4_xs(raw):
    b = np.asarray(raw, dtype=np.uint8).reshape(-1, 136)
    nb = b.shape[0]
    sub = np.arange(8)
    high = (np.ascontiguousarray(b[:, 2:4]).view('<u2').astype(np.int32) >> (2 * sub)[None, :]) & 3              # [nb, 8]
    low = np.stack([b[:, 4:8] & 0x0F, b[:, 4:8] >> 4], axis=2).reshape(nb, 8).astype(np.int32)                   # byte ib / 2, nibble ib % 2
    dl = (_half(b[:, 0:2]) * ((low | (high << 4)) - 32).astype(np.float32)).astype(np.float32)
    return (dl[:, :, None] * _nibble_values(b[:, 8:136].reshape(nb, 8, 16))).astype(np.float32).reshape(-1)


def iq2_s(raw, grid):
    """grid: uint8 [1024, 8], the format's codebook of magnitudes"""
    b = np.asarray(raw, dtype=np.uint8).reshape(-1, 82)
    nb = b.shape[0]
    two_bits = (b[:, 66:74, None] >> np.array([0, 2, 4, 6], np.uint8)) & 3                                       # [nb, 8, 4]: group g of sub-block ib
    index = b[:, 2:34].astype(np.int32) | (two_bits.reshape(nb, 32).astype(np.int32) << 8)
    mags = np.asarray(grid)[index].astype(np.float32)                                                           # [nb, 32, 8]
    minus = ((b[:, 34:66, None] >> np.arange(8, dtype=np.uint8)) & 1).astype(bool)                               # [nb, 32, 8]
    nib = np.stack([b[:, 74:82] & 0x0F, b[:, 74:82] >> 4], axis=2).reshape(nb, 16).astype(np.float32)            # a scale per 16 values
    db = ((_half(b[:, 0:2]) * (np.float32(0.5) + nib)).astype(np.float32) * np.float32(0.25)).astype(np.float32)  # [nb, 16]
    v = (np.repeat(db, 2, axis=1)[:, :, None] * mags).astype(np.float32)
    return np.where(minus, -v, v).astype(np.float32).reshape(-1)


DECODERS = {'Q4_K': (256, 144, q4_k), 'Q8_0': (32, 34, q8_0), 'IQ4_NL': (32, 18, iq4_nl), 'IQ4_XS': (256, 136, iq4_xs)}


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
