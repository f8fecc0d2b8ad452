"""Input generators shared by the CPU and GPU tests. The Q8 KV block sets restate the reference's fixed regression inputs
and its seeded generator (tests/io/test_own_kv_codec.py:24-68, seed 8103): data, not code under test."""
import numpy as np


def _bits(word):
    return np.array([word], np.uint32).view(np.float32)[0]


def kv_valid_blocks():
    f = np.float32
    rows = []

    def add(vals):
        r = np.zeros(32, f); r[:len(vals)] = vals; rows.append(r)

    add([0, -0.0])
    add([127, .5, -.5, 1.5, -1.5, 2.5, -2.5, np.nextafter(f(.5), f(0)), -np.nextafter(f(.5), f(0)), np.nextafter(f(.5), f(1))])
    add([_bits(0x42fe1382), _bits(0x427e0a3d), -_bits(0x427e0a3d)])
    for scale in (0x3f801000, 0x3f803000):
        add([_bits(scale) * f(127)])
    add([3, _bits(0x3c418306), -_bits(0x3c418306)])
    add([f(1.27e-6), -f(1.27e-6)])
    add([f(127 * 2 ** -24), -f(127 * 2 ** -24)])
    for e in (-121, -120):
        add([f(2.0 ** e), -f(2.0 ** e)])
    add([f(127 * 65504), -f(127 * 65504)])
    add([np.nextafter(f(65520), f(0)) * f(127)])
    rng = np.random.default_rng(8103)
    rnd = rng.uniform(-1, 1, size=(4096, 32)).astype(f)
    rnd *= np.exp2(rng.integers(-90, 23, size=(4096, 1))).astype(f)
    return np.ascontiguousarray(np.concatenate((np.stack(rows), rnd)))


def kv_invalid_blocks():
    f = np.float32
    rows = []
    for value in (np.nan, np.inf, -np.inf, np.finfo(f).max, np.nextafter(f(0), f(1)), f(2 ** -128), f(65520 * 127)):
        r = np.zeros(32, f); r[-1] = value; rows.append(r)
    return np.stack(rows)


def q4k_table(rng, rows, N):
    """random Q4_K rows: every nibble / 6-bit scale pattern, fp16 d, dmin ~ U(1e-3, 1e-2); uint8 [rows, N / 256 * 144]"""
    nb = N // 256
    t = rng.integers(0, 256, (rows, nb, 144), dtype=np.uint8)
    dd = rng.uniform(1e-3, 1e-2, (rows, nb, 2)).astype(np.float16)
    t[:, :, 0:4] = dd.view(np.uint8).reshape(rows, nb, 4)
    return t.reshape(rows, nb * 144)


def q80_table(rng, rows, N):
    """random Q8_0 rows: codes U{-128..127}, fp16 d ~ U(1e-3, 1e-2); uint8 [rows, N / 32 * 34]"""
    nb = N // 32
    t = rng.integers(0, 256, (rows, nb, 34), dtype=np.uint8)
    dd = rng.uniform(1e-3, 1e-2, (rows, nb, 1)).astype(np.float16)
    t[:, :, 0:2] = dd.view(np.uint8).reshape(rows, nb, 2)
    return t.reshape(rows, nb * 34)


def iq_table(rng, rows, N, fmt):
    """random IQ4_XS / IQ2_S / IQ4_NL rows: every index, sign and scale pattern, fp16 d ~ N(0, 0.01) (either sign);
    uint8 [rows, N / values * bytes]"""
    qk, bs = {'IQ4_XS': (256, 136), 'IQ2_S': (256, 82), 'IQ4_NL': (32, 18)}[fmt]
    nb = N // qk
    t = rng.integers(0, 256, (rows, nb, bs), dtype=np.uint8)
    t[:, :, 0:2] = (rng.standard_normal((rows, nb, 1)) * 0.01).astype(np.float16).view(np.uint8).reshape(rows, nb, 2)
    return t.reshape(rows, nb * bs)


def qk_par(rng, theta_base=1e6, eps=1e-6, yarn_table=None):
    """the own line's par block: q_norm[128] | k_norm[128] | theta_scale | eps (| freq[64] | mscale)"""
    qn = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32); kn = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    ts = np.float32(np.float32(theta_base) ** np.float32(-2.0 / 128))
    par = np.concatenate([qn, kn, np.array([ts, eps], np.float32)])
    if yarn_table is not None: par = np.concatenate([par, np.asarray(yarn_table, np.float32)])
    return par.astype(np.float32)
