"""Pins of the CPU oracle (oracle/camx_oracle.c) that do not restate its own formulas: the reference's literal byte
vectors and seeded generators, the reference's own header compiled for the host (oracle/_ref, when it was built here),
independent numpy implementations written from the format definitions, float64 closed forms, and invariants chosen so that
a dropped term, a wrong index or a transposed operand fails. CPU only."""
import math
import os

import numpy as np
import pytest

import oracle as O
from caminus_amd import rope
from oracle import np_dequant as own_dequant, np_kv as ref_kv
from vectors import iq_table, kv_invalid_blocks, kv_valid_blocks, q4k_table, q80_table, qk_par

f32 = np.float32


def _bits(word):
    return np.array([word], np.uint32).view(np.float32)[0]


# ---- conversions ----------------------------------------------------------------------------------------------------------

def test_fp16_conversions_match_numpy_everywhere():
    allh = np.arange(65536, dtype=np.uint16)
    got, want = O.h2f(allh), allh.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok]) and np.isnan(got[~ok]).all()
    fin = allh[(allh & 0x7c00) != 0x7c00].view(np.float16).astype(np.float32)
    mids = ((fin.astype(np.float64) + np.roll(fin, -1).astype(np.float64)) / 2).astype(np.float32)       # ties and their neighbours
    rng = np.random.default_rng(0)
    rnd = rng.standard_normal(200000).astype(f32) * np.exp2(rng.integers(-30, 18, 200000)).astype(f32)
    for x in (mids, np.nextafter(mids, f32(np.inf)), np.nextafter(mids, f32(-np.inf)), rnd,
              np.array([0, -0.0, 65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, np.inf, -np.inf], f32)):
        with np.errstate(over='ignore'):
            assert np.array_equal(O.f2h(x), x.astype(np.float16).view(np.uint16))


def test_bf16_rounding_is_nearest_even_with_nan_canonicalised():
    x = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, np.finfo(np.float32).max, np.inf, -np.inf, np.nan, 1e-40], f32)
    # 1 + 2^-8 is a tie -> even (1.0); 1 + 3 * 2^-8 is a tie -> even (1 + 2^-6); max finite rounds to inf
    assert O.f2bf(x).tolist() == [0x3f80, 0x3f80, 0x3f82, 0xbf80, 0x7f80, 0x7f80, 0xff80, 0x7fc0, 0x0001]
    rng = np.random.default_rng(1)
    r = rng.standard_normal(100000).astype(f32)
    back = O.bf2f(O.f2bf(r))
    assert (np.abs(back - r) <= np.abs(r) * 2.0 ** -8).all() and np.array_equal(O.f2bf(back), O.f2bf(r))


# ---- Q8 KV wire block: the reference's fixed vectors (tests/io/test_ref_kv.py:39-94) -----------------------------------------

def _blk(scale_bytes, codes):
    return bytes(scale_bytes) + np.array(codes + [0] * (32 - len(codes)), np.int8).tobytes()


KV_LITERALS = [
    # (values, stored half scale bytes, codes): ties away from zero and the floats adjacent to a tie
    ([127, .5, -.5, 1.5, -1.5, 2.5, -2.5, np.nextafter(f32(.5), f32(0)), -np.nextafter(f32(.5), f32(0)), np.nextafter(f32(.5), f32(1)),
      -np.nextafter(f32(.5), f32(1))], [0, 0x3c], [127, 1, -1, 2, -2, 3, -3, 0, 0, 1, -1]),
    # the stored half scale rounds to 1 while the fp32 scale gives code 63 (the half scale would give 64)
    ([_bits(0x42fe1382), _bits(0x427e0a3d), -_bits(0x427e0a3d)], [0, 0x3c], [127, 63, -63]),
    # half scale ties round to even at both neighbours
    ([_bits(0x3f801000) * f32(127)], [0x00, 0x3c], [127]),
    ([_bits(0x3f803000) * f32(127)], [0x02, 0x3c], [127]),
    # x / d is exactly .5 but x * fp32(1 / d) is the float just below .5
    ([3, _bits(0x3c418306), -_bits(0x3c418306)], [0x0c, 0x26], [127, 0, 0]),
    # a normal fp32 scale that rounds to stored half zero: the codes survive
    ([f32(1.27e-6), -f32(1.27e-6), 0], [0, 0], [127, -127, 0]),
    # the smallest half subnormal scale
    ([f32(127 * 2 ** -24), -f32(127 * 2 ** -24), 0], [1, 0], [127, -127, 0]),
]


@pytest.mark.parametrize('vals,scale,codes', KV_LITERALS)
def test_kv_q8_literal_blocks(vals, scale, codes):
    x = np.zeros(32, f32); x[:len(vals)] = vals
    raw, ok = O.kv_q8_encode(x[None])
    assert ok[0] == 1 and raw[0].tobytes() == _blk(scale, codes)


def test_kv_q8_row_layout_and_chunking():
    """K then V, head-major, distinct scales per (row, part, head) make the order observable (test_ref_kv.py:96-124)"""
    for heads, dim in ((1, 128), (1, 256), (3, 128), (3, 256)):
        M = heads * dim
        signed = np.tile(np.array([-127, 127, -1, 1] + [0] * 28, f32), dim // 32)
        fac = np.arange(1, 3 * heads + 1, dtype=f32).reshape(3, heads, 1)
        k = (signed * fac).reshape(3, M); v = k * f32(2)
        cache, err = O.kv_q8_append(k, M, v, M, M, np.zeros(3 * 2 * (M // 32) * 34, np.uint8), 0, 3)
        want = b''
        for row in range(3):
            for mult in (1, 2):
                for h in range(heads):
                    s = np.array([(row * heads + h + 1) * mult], '<f2').view(np.uint8).tolist()
                    want += _blk(s, [-127, 127, -1, 1]) * (dim // 32)
        assert err == 0 and cache.tobytes() == want
        # the independent numpy codec agrees on the same rows
        lay = ref_kv.Q8KVLayout(heads, dim)
        assert ref_kv.encode_q8_kv(k.reshape(3, heads, dim), v.reshape(3, heads, dim), lay).tobytes() == want


def test_kv_q8_generator_blocks_against_compiled_reference_and_numpy():
    good, bad = kv_valid_blocks(), kv_invalid_blocks()
    raw, ok = O.kv_q8_encode(np.concatenate([good, bad]))
    assert ok[:len(good)].all() and not ok[len(good):].any()
    assert (raw[len(good):] == 0xa5).all()                                    # refused blocks keep their bytes
    even = good[:len(good) // 2 * 2]
    want = ref_kv.encode_q8_kv(even[::2, None, :], even[1::2, None, :], ref_kv.Q8KVLayout(1, 32)).reshape(-1, 34)
    assert np.array_equal(raw[:len(even)].reshape(-1, 2, 34).reshape(-1, 34), np.stack([want[0::2], want[1::2]], 1).reshape(-1, 34))
    for b in bad:
        with pytest.raises(ValueError):
            ref_kv.encode_q8_kv(b[None, None, :], b[None, None, :], ref_kv.Q8KVLayout(1, 32))
    ref = O.ref_kv_q8_encode(np.concatenate([good, bad]))
    if ref is None:
        pytest.skip('oracle/_ref was not built in this checkout (the reference source is absent)')
    assert np.array_equal(ref[0], raw) and np.array_equal(ref[1], ok)


def test_kv_q8_error_bits():
    k = np.ones((4, 64), f32)
    z = np.full(4 * 136, 0xa5, np.uint8)
    assert O.kv_q8_append(k, 64, k, 64, 64, z, 0, 4)[1] == 0
    assert O.kv_q8_append(k, 64, k, 64, 64, z, 2, 4, rows=4)[1] == 1            # rows 4, 5 outside
    assert O.kv_q8_append(k, 64, k, 64, 48, z, 0, 4, rows=4)[1] == 4            # M % 32
    assert O.kv_q8_append(k, 63, k, 64, 64, z, 0, 4, rows=4)[1] == 4            # ld < M
    kb = k.copy(); kb[1, 5] = np.inf
    cache, err = O.kv_q8_append(kb, 64, k, 64, 64, z, 0, 4)
    assert err == 2 and (cache.reshape(4, 4, 34)[1, 0] == 0xa5).all() and not (cache.reshape(4, 4, 34)[1, 1] == 0xa5).all()


# ---- Hadamard ---------------------------------------------------------------------------------------------------------------

def _sylvester(n):
    H = np.array([[1.0]])
    while H.shape[0] < n: H = np.block([[H, H], [H, -H]])
    return H / math.sqrt(n)


def test_hadamard128_against_float64_sylvester():
    rq = np.random.default_rng(8)
    xs = np.concatenate([rq.standard_normal((40, 128)), rq.standard_normal((8, 128)) * 1e3, np.eye(128)[:8] * 65504,
                         rq.standard_normal((8, 128)) * np.where(np.arange(128) % 17 == 0, 60.0, 0.1)]).astype(f32)
    H = _sylvester(128)
    hx = O.hadamard128(xs)
    assert (np.abs(hx - xs.astype(np.float64) @ H.T).max(1) / np.abs(xs).max(1)).max() < 2e-6
    assert np.float32(float.fromhex('0x1.6a09e6p-4')) == np.float32(1 / np.sqrt(128))
    # unit spikes read a column of H: exact signs, every magnitude the scale itself
    e = O.hadamard128(np.eye(128, dtype=f32))
    assert np.array_equal(np.sign(e), np.sign(H)) and (np.abs(e) == np.float32(float.fromhex('0x1.6a09e6p-4'))).all()
    # the rotation keeps scores: (H q) . (H k) = q . k
    q, k = rq.standard_normal((64, 128)).astype(f32), rq.standard_normal((64, 128)).astype(f32)
    s0 = (q.astype(np.float64) * k).sum(1); s1 = (O.hadamard128(q).astype(np.float64) * O.hadamard128(k)).sum(1)
    assert np.abs(s1 - s0).max() < 1e-4
    assert np.array_equal(hx, ref_kv.hadamard128(xs))                          # the independent numpy butterflies, bit for bit


def test_hadamard128_lane_by_lane_emulation():
    """the reference kernel's own data layout (lane l holds dims l, l + 32, l + 64, l + 96; shuffle stages h = 1 .. 16, then
    32 and 64 in registers: tests/engine/test_q3moe_kvq8_cpu.py:176-197) gives the same bits as the sequential butterflies"""
    rq = np.random.default_rng(9)
    xs = (rq.standard_normal((16, 128)) * 3).astype(f32)
    sc = np.float32(float.fromhex('0x1.6a09e6p-4'))
    out = np.empty_like(xs)
    lanes = np.arange(32)
    for r, x in enumerate(xs):
        for qw in range(4):
            u = [x[lanes + 32 * m].copy() for m in range(4)]
            h = 1
            while h < 32:
                hi = (lanes & h) != 0
                u = [np.where(hi, um[lanes ^ h] - um, um + um[lanes ^ h]).astype(f32) for um in u]
                h *= 2
            a0, a1, a2, a3 = u[0] + u[1], u[0] - u[1], u[2] + u[3], u[2] - u[3]
            out[r, 32 * qw:32 * qw + 32] = ((a0 + a2, a1 + a3, a0 - a2, a1 - a3)[qw] * sc).astype(f32)
    assert np.array_equal(out, O.hadamard128(xs))


@pytest.mark.parametrize('n', [64, 128, 256])
def test_hadamard_n(n):
    rq = np.random.default_rng(n)
    x = rq.standard_normal((11, n)).astype(f32)
    y = O.hadamard_n(x, n)
    assert np.abs(y - x.astype(np.float64) @ _sylvester(n).T).max() < 1e-5
    assert np.abs(O.hadamard_n(y, n) - x).max() < 1e-5                          # an involution
    if n != 128: assert np.array_equal(O.hadamard_n(np.eye(n, dtype=f32)[:3], n), (_sylvester(n)[:3]).astype(f32))   # power-of-two scale: exact


# ---- GGUF rows: scalar per-value definitions (tests/io/test_own_formats.py:31-68) -----------------------------------------------

def _fp16_at(b, o):
    return f32(np.frombuffer(bytes(b[o:o + 2]), np.float16)[0])


def _k_scale_min(s, j):
    if j < 4: return s[j] & 63, s[j + 4] & 63
    return (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4)


def _def_q4_k(b, i):
    d, dmin, s, qs = _fp16_at(b, 0), _fp16_at(b, 2), b[4:16], b[16:144]
    j, n, l = i // 32, i // 64, i % 32
    sc, m = _k_scale_min(s, j)
    q = (qs[n * 32 + l] >> 4) if j % 2 else (qs[n * 32 + l] & 0xF)
    return (d * f32(sc)) * f32(q) - dmin * f32(m)


def _def_q8_0(b, i):
    return _fp16_at(b, 0) * f32(np.frombuffer(bytes(b[2:34]), np.int8)[i])


def test_gguf_rows_against_scalar_definitions():
    rng = np.random.default_rng(5)
    N, vocab = 512, 6
    t4 = q4k_table(rng, vocab, N); t4[0] = 0; t4[1, 4:] = 255
    toks = np.array([5, 0, 1, -3, 99, 2], np.int32)                                # clamped: -3 -> 0, 99 -> 5
    x, xbf = O.emb_q4k(t4, vocab, toks, N)
    with np.errstate(over='ignore', invalid='ignore'):
        for r, tk in enumerate(np.clip(toks, 0, vocab - 1)):
            row = t4[tk]
            want = np.array([_def_q4_k(row[(i // 256) * 144:(i // 256 + 1) * 144], i % 256) for i in range(N)], f32)
            assert np.array_equal(x[r].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(xbf, O.f2bf(x))
    assert np.array_equal(x[0].view(np.uint32), own_dequant.q4_k(t4[5]).view(np.uint32))
    t8 = q80_table(rng, vocab, N)
    y, ybf = O.emb_q8_0(t8, vocab, toks, N)
    for r, tk in enumerate(np.clip(toks, 0, vocab - 1)):
        row = t8[tk]
        want = np.array([_def_q8_0(row[(i // 32) * 34:(i // 32 + 1) * 34], i % 32) for i in range(N)], f32)
        assert np.array_equal(y[r].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(ybf, O.f2bf(y))


KV_IQ4 = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]      # ggml's kvalues_iq4nl (kernels/prefill_feed.hip:15)


def test_iq2s_codebook_file():
    """the codebook is format data that cannot be derived: its bytes are held to a digest and to the entries the format's
    published table starts with; every entry is 8 magnitudes out of {8, 25, 43} and no entry repeats"""
    import hashlib
    g = O.iq2s_grid()
    assert g.shape == (1024, 8) and g.dtype == np.uint8
    assert hashlib.sha256(g.tobytes()).hexdigest() == 'e1aa1473412b0552c2174c30ef22ab4073f6a181b85a17056e8249bd2932fd88'
    assert g[0].tolist() == [8] * 8 and g[1].tolist() == [43] + [8] * 7 and g[2].tolist() == [25, 25] + [8] * 6
    assert set(np.unique(g).tolist()) == {8, 25, 43} and len({bytes(r) for r in g}) == 1024
    # the product's copy (little-endian words of four magnitudes) holds the same bytes
    import re
    txt = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'caminus_amd', 'csrc', 'iq2s_grid.inc')).read()
    words = np.array([int(w, 16) for w in re.findall(r'0x([0-9a-f]{8})u', txt)], np.uint32)
    assert np.array_equal(words.view(np.uint8).reshape(1024, 8), g)


def test_iq_rows_known_answers():
    """hand-built blocks whose values are known without any decoder"""
    h = lambda v: np.array([v], np.float16).view(np.uint8)
    # IQ4_NL, d = 1: byte i holds index i (low nibble) and 15 - i (high): values 0-15 ascend through the table, 16-31 descend
    blk = np.zeros(18, np.uint8); blk[0:2] = h(1.0); blk[2:18] = np.arange(16) | ((15 - np.arange(16)) << 4)
    out, err = O.ple_rows_iq4nl(blk[None], np.array([0], np.int32), 1, 1)
    assert err == 0 and out[0].tolist() == KV_IQ4 + KV_IQ4[::-1]
    assert np.array_equal(own_dequant.iq4_nl(blk), out[0])
    # IQ4_XS, d = 2, sub-block ib has the 6-bit scale 33 + ib (low nibble 1 + ib, high bits 2), every index 8 (value 1) but two
    blk = np.zeros(136, np.uint8); blk[0:2] = h(2.0)
    blk[2:4] = np.array([sum(2 << (2 * ib) for ib in range(8))], np.uint16).view(np.uint8)
    blk[4:8] = [(1 + 2 * k) | ((2 + 2 * k) << 4) for k in range(4)]
    blk[8:136] = 0x88
    blk[8 + 16 * 3 + 5] = 0x0F                                           # sub-block 3: value 5 -> index 15, value 21 -> index 0
    x, _, err = O.emb_iq4xs(blk[None], 1, np.array([0], np.int32), 256)
    want = np.repeat(2.0 * (1 + np.arange(8)), 32).astype(f32); want[3 * 32 + 5] *= 113; want[3 * 32 + 21] *= -127
    assert err == 0 and np.array_equal(x[0], want)
    # IQ2_S, d = 4: db = 0.5 + s; sub-block 2 / group 1 (values 72-79) points at codebook entry 0x101 + signs 0b10000001
    g = O.iq2s_grid()
    blk = np.zeros(82, np.uint8); blk[0:2] = h(4.0)
    blk[2 + 4 * 2 + 1] = 0x01; blk[66 + 2] = 1 << 2; blk[34 + 9] = 0x81
    blk[74:82] = [0x10 * (k + 1) | k for k in range(8)]                 # 16-value halves of sub-block k: scales k and k + 1
    x, _ = O.emb_iq2s(blk[None], 1, np.array([0], np.int32), 256)
    want = np.repeat(0.5 + np.stack([np.arange(8), np.arange(8) + 1], 1).reshape(-1), 16).astype(f32) * 8       # entry 0: all 8
    want[72:80] = 2.5 * g[0x101].astype(f32) * np.array([-1, 1, 1, 1, 1, 1, 1, -1], f32)
    assert np.array_equal(x[0], want)


def test_iq_rows_against_block_decoders():
    """the one-value-at-a-time C statements against the block-wise numpy decoders on random blocks (both signs of d, every bit
    pattern), with clamped ids and the error word"""
    rng = np.random.default_rng(15)
    vocab, toks = 7, np.array([3, 0, 6, 9, -2, 5], np.int32)
    rows = np.clip(toks, 0, vocab - 1)
    for N in (256, 768, 2048):
        W = iq_table(rng, vocab, N, 'IQ4_XS')
        x, xbf, err = O.emb_iq4xs(W, vocab, toks, N)
        assert err == 2 and np.array_equal(x.view(np.uint32), own_dequant.iq4_xs(W.reshape(-1)).reshape(vocab, N)[rows].view(np.uint32))
        assert np.array_equal(xbf, O.f2bf(x)) and O.emb_iq4xs(W, vocab, rows, N)[2] == 0
        W = iq_table(rng, vocab, N, 'IQ2_S')
        x, xbf = O.emb_iq2s(W, vocab, toks, N)
        assert np.array_equal(x.view(np.uint32), own_dequant.iq2_s(W.reshape(-1), O.iq2s_grid()).reshape(vocab, N)[rows].view(np.uint32))
        assert np.array_equal(xbf, O.f2bf(x))
    for bpr in (1, 5, 8):
        raw = iq_table(rng, 4, 32 * bpr, 'IQ4_NL'); inv = np.array([0, 3, 1, 4, -1, 2], np.int32)
        out, err = O.ple_rows_iq4nl(raw, inv, 4, bpr)
        assert err == 1 and np.array_equal(out.view(np.uint32), own_dequant.iq4_nl(raw.reshape(-1)).reshape(4, 32 * bpr)[np.clip(inv, 0, 3)].view(np.uint32))


# ---- q8_1 -------------------------------------------------------------------------------------------------------------------------

def _q8_host(x):
    """the reference's host model of quantize_q8_1 (tests/engine/golden_util.py:101-110)"""
    xb = np.asarray(x, f32).reshape(-1, 32); amax = np.abs(xb).max(1); d = (amax / f32(127.0)).astype(f32)
    with np.errstate(divide='ignore', invalid='ignore'):
        v = np.where(d[:, None] > 0, xb / np.where(d > 0, d, 1)[:, None], 0).astype(f32)
    return d.astype(np.float16), (np.sign(v) * np.floor(np.abs(v.astype(np.float64)) + 0.5)).astype(np.int8)


def _tree32(v):
    """the 32-lane xor butterfly written as explicit halving levels"""
    v = np.asarray(v, f32)
    for o in (16, 8, 4, 2, 1):
        v = (v[:o] + v[o:2 * o]).astype(f32)
    return v[0]


def test_q8_1_blocks():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(64 * 32) * np.exp2(rng.integers(-8, 8, 64 * 32))).astype(f32)
    x[:32] = 0; x[32:64] = 127 * np.sign(rng.standard_normal(32)); x[64:96] = np.arange(32) + 0.5      # zero block, full scale, ties
    y = O.q8_1(x)
    d, q = _q8_host(x)
    assert np.array_equal(y[:, 0:2].copy().view(np.float16).reshape(-1), d) and np.array_equal(y[:, 4:].view(np.int8), q)
    assert not y[0].any()                                                          # all-zero block: d = 0, sum = 0, codes 0
    assert y[1, 0:2].copy().view(np.float16)[0] == 1.0 and (np.abs(y[1, 4:].view(np.int8)) == 127).all()
    s = y[:, 2:4].copy().view(np.float16).reshape(-1)
    assert np.array_equal(s, np.array([_tree32(b) for b in x.reshape(-1, 32)], f32).astype(np.float16))
    # the tree order is observable: one large value cancels against its partner only under the butterfly pairing
    v = np.zeros(32, f32); v[0] = 2.0 ** 24; v[16] = -2.0 ** 24; v[1] = 1.0; v[2] = 1.0
    assert O.lib().orc_bfly32_sum(v.ctypes.data) == 2.0 and np.float32(np.cumsum(v, dtype=f32)[-1]) != 2.0
    # tail: values past n quantize as 0 and the last block is still written
    t = O.q8_1(x[:40])
    assert t.shape == (2, 36) and np.array_equal(t[0], y[0]) and not t[1, 4 + 8:].any()


def test_q8_codes_when_the_scale_underflows_and_blocks_of_nan():
    """known answers for the two statements that C leaves open: a quotient outside the int8 range takes the saturating
    float -> int32 conversion's low byte (+inf -> 0x7fffffff -> -1, -inf -> 0x80000000 -> 0, NaN -> 0), and a block of NaNs has
    amax 0 (fmaxf skips a NaN)"""
    tiny = np.float32(1e-44)                                               # a subnormal: tiny / 127 rounds to 0, so x / d = +-inf
    x = np.zeros(3 * 32, f32); x[0] = tiny; x[1] = -tiny; x[2] = tiny / 2
    x[32:64] = np.nan
    x[64] = np.nan; x[65] = 3.0; x[66] = -1.5
    y = O.q8_1(x)
    assert y[0, 0] == 0 and y[0, 1] == 0                                   # d = 0
    assert y[0, 4:8].view(np.int8).tolist() == [-1, 0, -1, 0]              # +inf, -inf, +inf, 0 / 0 = NaN
    assert not y[1, :2].any() and not y[1, 4:].any()                       # the block of NaNs: scale 0, codes 0
    assert y[2, 0:2].copy().view(np.float16)[0] == np.float16(f32(3.0) / f32(127.0)) and y[2, 4:7].view(np.int8).tolist() == [0, 127, -64]
    # MMQ layout: 127 / amax overflows for amax below 127 / FLT_MAX
    K = 128
    xm = np.zeros((1, K), f32); xm[0, 0] = f32(1e-38) / 64; xm[0, 1] = -xm[0, 0]
    b = O.mmq_q8_1(xm, K, 1, 0)[0, 0]
    assert b[:4].copy().view(f32)[0] == 0.0 and b[16:19].view(np.int8).tolist() == [-1, 0, 0]      # d = 1 / inf = 0; +inf, -inf, 0 * inf
    assert O.set_threads(1) >= 1 and O.set_threads(0) == 1                 # (the thread control of the timing leg: previous setting returned)


def test_mmq_q8_1_layout_and_invariants():
    rng = np.random.default_rng(4)
    K, ncols = 640, 5
    x = (rng.standard_normal((ncols, K)) * 3).astype(f32); x[2, :32] = 0
    y4, ys = O.mmq_q8_1(x, K, ncols, 0), O.mmq_q8_1(x, K, ncols, 1)
    assert y4.shape == (O.k_pad(K) // 128, ncols, 144) == (8, 5, 144)
    assert np.array_equal(y4[:, :, 16:], ys[:, :, 16:])                           # the codes do not depend on the header layout
    for c in range(ncols):
        for kb in range(8):
            q = ys[kb, c, 16:].view(np.int8).astype(np.float64).reshape(4, 32)
            d4 = y4[kb, c, :16].copy().view(np.float32)
            ds = ys[kb, c, :16].copy().view(np.float16).reshape(4, 2)
            seg = np.zeros(128, f32); lo = kb * 128
            if lo < K: seg[:min(128, K - lo)] = x[c, lo:lo + 128]
            seg = seg.reshape(4, 32)
            assert np.array_equal(ds[:, 0], d4.astype(np.float16))
            assert (np.abs(q * d4[:, None] - seg) <= d4[:, None] * 0.5 * (1 + 1e-6) + 1e-12).all()       # reconstruction within half a step
            assert np.allclose(ds[:, 1].astype(np.float64), seg.sum(1), rtol=2e-3, atol=2e-3)
            if lo >= K: assert not ys[kb, c].any()                                 # K padding: zeros, d = 0
    assert not ys[0, 2, 16:48].any() and ys[0, 2, 0:4].view(np.uint32)[0] == 0     # an all-zero group
    ids = np.array([4, 0, 2], np.int32)
    g = O.mmq_q8_1(x, K, 3, 1, ids=ids)
    assert np.array_equal(g, ys[:, ids])
    inv = np.array([5, 1, 0, 4, 3, 2], np.int32)                                    # 3 tokens x 2 slots
    sc = O.mmq_q8_1_scatter(x[:3], K, 3, inv, 2, 1)
    for t in range(3):
        for s in range(2): assert np.array_equal(sc[:, inv[2 * t + s]], ys[:, t])


def test_mmq_q8_1_bit_level_known_answers():
    """what the vendored statement (kernels/ggml_mmq/quantize_mmq.cuh:78-112) fixes to the last bit and a plausible restatement would
    get wrong: ties away from zero; codes from x * (127 / amax), not x / (amax / 127); d = 1 / (127 / amax), not amax / 127; and the
    DS4 sum as ((x0 + x1) + x2) + x3 per thread, then thread xor 4, 2, 1"""
    K = 128

    def block(v32, layout):
        x = np.zeros((1, K), f32); x[0, :32] = v32
        b = O.mmq_q8_1(x, K, 1, layout)[0, 0]
        hdr = b[:4].copy()
        return (hdr.view(f32)[0] if layout == 0 else hdr.view(np.float16)), b[16:48].view(np.int8)

    # amax = 127: 127 / amax = 1 exactly, the codes are roundf(x): halves go away from zero
    v = np.zeros(32, f32); v[0] = 127; v[1:13] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.49999997, 126.5, -126.5, 3.5, 4.5]
    d, q = block(v, 0)
    assert d == 1.0 and q[:13].tolist() == [127, 1, -1, 2, -2, 3, -3, 0, 0, 127, -127, 4, 5]
    # a value whose product with fl(127 / amax) and whose quotient by fl(amax / 127) round to different codes: found by a seeded
    # search over values next to a tie
    rng = np.random.default_rng(12)
    found = None
    for _ in range(400):
        amax = rng.uniform(1, 4, 20000).astype(f32); k = rng.integers(1, 126, 20000)
        x = ((k + 0.5) * (amax.astype(np.float64) / 127.0)).astype(f32)                 # near a tie
        pm = (x * (f32(127.0) / amax)).astype(f32); pd = (x / (amax / f32(127.0))).astype(f32)
        rm = np.sign(pm) * np.floor(np.abs(pm.astype(np.float64)) + 0.5); rd = np.sign(pd) * np.floor(np.abs(pd.astype(np.float64)) + 0.5)
        hit = np.nonzero((rm != rd) & (x <= amax))[0]
        if hit.size: found = (amax[hit[0]], x[hit[0]], int(rm[hit[0]]), int(rd[hit[0]])); break
    assert found is not None
    amax, x, by_mul, by_div = found
    v = np.zeros(32, f32); v[0] = amax; v[1] = x; v[2] = -x
    d, q = block(v, 0)
    assert by_mul != by_div and q[1] == by_mul and q[2] == -by_mul and q[0] == 127
    # d is the reciprocal of the reciprocal: an amax where fl(1 / fl(127 / amax)) differs from fl(amax / 127)
    cand = rng.uniform(0.5, 8, 200000).astype(f32)
    two = (f32(1.0) / (f32(127.0) / cand)).astype(f32); one = (cand / f32(127.0)).astype(f32)
    amax = cand[np.nonzero(two != one)[0][0]]
    v = np.zeros(32, f32); v[5] = -amax
    d, q = block(v, 0)
    assert d == f32(1.0) / (f32(127.0) / amax) and d != amax / f32(127.0) and q[5] == -127
    ds, _ = block(v, 1)
    assert ds[0] == np.float16(d) and ds[1] == np.float16(-amax)
    # the DS4 sum. Thread t holds values 4t .. 4t + 3. (a) inside a thread: ((2^24 + 1) + 1) + -2^24 = 0 (each 1 is lost), any other
    # association gives 1 or 2
    v = np.zeros(32, f32); v[0:4] = [2.0 ** 24, 1, 1, -2.0 ** 24]
    assert block(v, 1)[0][1] == 0.0
    v[0:4] = [2.0 ** 24, -2.0 ** 24, 1, 1]
    assert block(v, 1)[0][1] == 2.0
    # (b) across threads: partners are t ^ 4 first. Thread sums s0 = 2^24, s4 = 1, s2 = 1, s6 = -2^24:
    # (s0 + s4) + (s2 + s6) = 2^24 + -(2^24 - 1) = 1; pairing neighbours first ((s0 + s2) + (s4 + s6)) would also lose a 1 but a
    # running sum over threads 0 .. 7 gives 2^24 + 1 + 1 - 2^24 = 0
    v = np.zeros(32, f32); v[0] = 2.0 ** 24; v[16] = 1; v[8] = 1; v[24] = -2.0 ** 24
    assert block(v, 1)[0][1] == 1.0
    # partners t ^ 4 then t ^ 2 then t ^ 1: s0 = 2^24, s1 = -2^24, s4 = 1, s5 = 1 -> ((s0 + s4) + 0) + ((s1 + s5) + 0) = 2^24 + -(2^24 - 1) = 1,
    # where xor 1 first would give (s0 + s1) + (s4 + s5) = 2
    v = np.zeros(32, f32); v[0] = 2.0 ** 24; v[4] = -2.0 ** 24; v[16] = 1; v[20] = 1
    assert block(v, 1)[0][1] == 1.0


# ---- RMSNorm family ---------------------------------------------------------------------------------------------------------------

def test_dense_line_h16_is_the_last_product_rounded_once():
    """q35p_add_rms16's fp16 copy: the reference's binary rounds it straight from the last product (kernels/q35_prefill.hip:630-635), so the
    oracle rounds the exact product once. Known answer: (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24 lies above the fp16 tie at 1 + 2^-11 and goes to
    0x3c01, where fp32 first (ties to even: 1 + 2^-11) and fp16 second (ties to even: 1.0) give 0x3c00. The conversion itself against
    numpy's double -> half on random products, subnormal and overflowing ones included."""
    import ctypes as C
    L = O.lib(); L.orc_mul_f2h_once.restype = C.c_uint16; L.orc_mul_f2h_once.argtypes = [C.c_float, C.c_float]
    a = f32(1 + 2.0 ** -12)
    assert L.orc_mul_f2h_once(a, a) == 0x3c01 and O.f2h(np.array([a * a], f32))[0] == 0x3c00
    assert L.orc_mul_f2h_once(f32(-0.0), f32(3.0)) == 0x8000 and L.orc_mul_f2h_once(f32(300.0), f32(300.0)) == 0x7c00
    rng = np.random.default_rng(21)
    x = (rng.standard_normal(20000) * np.exp2(rng.integers(-20, 12, 20000))).astype(f32); y = (rng.standard_normal(20000) * np.exp2(rng.integers(-12, 8, 20000))).astype(f32)
    with np.errstate(over='ignore'):
        want = (x.astype(np.float64) * y.astype(np.float64)).astype(np.float16).view(np.uint16)
    assert np.array_equal(np.array([L.orc_mul_f2h_once(float(p), float(q)) for p, q in zip(x, y)], np.uint16), want)
    # the row function uses it: h16 = half(exact(fl(x scale) nw)), h = fl of the same product; the scale from the sibling pf_rms_mul
    n, N = 3, 2560
    xr = (rng.standard_normal((n, N)) * 3).astype(f32); nw = (1 + 0.1 * rng.standard_normal(N)).astype(f32)
    r = O.add_rms16_q35(xr, nw, 1e-6)
    t = (xr * O.rms_mul(xr, nw, 1e-6)['scale'][:, None]).astype(f32)
    assert np.array_equal(r['h'], (t * nw).astype(f32))
    assert np.array_equal(r['h16'], (t.astype(np.float64) * nw.astype(np.float64)).astype(np.float16).view(np.uint16))
    assert (r['h16'] != O.f2h(r['h'])).sum() < n * N * 1e-3                # (one value in about 16000 differs from the twice-rounded one)


def test_add_rms_closed_form_and_invariants():
    rng = np.random.default_rng(6)
    n, N, S = 5, 2048, 3
    x = rng.standard_normal((n, N)).astype(f32); d = rng.standard_normal((n, S, N)).astype(f32); w = rng.random((n, S)).astype(f32)
    nw = (1 + 0.1 * rng.standard_normal(N)).astype(f32)
    r = O.add_rms16(x, nw, 1e-6, d=d, w=w, S=S, want_q8=True)
    xx = x.astype(np.float64) + (w[:, :, None].astype(np.float64) * d).sum(1)
    want = xx / np.sqrt((xx * xx).mean(1, keepdims=True) + 1e-6) * nw
    assert np.abs(r['x'] - xx).max() < 1e-5 and np.abs(r['h'] - want).max() < 1e-5 * np.abs(want).max()
    assert np.array_equal(r['h16'], O.f2h(r['h'])) and np.array_equal(r['q8'].reshape(-1, 36), O.q8_1(r['h']))
    # gamma = 1 gives unit RMS rows; scaling x by 2^k scales nothing (eps aside)
    one = O.add_rms16(x, np.ones(N, f32), 0.0)
    assert np.allclose((one['h'].astype(np.float64) ** 2).mean(1), 1.0, atol=1e-5)
    assert np.array_equal(O.add_rms16(x * f32(4), np.ones(N, f32), 0.0)['h'], one['h'])
    # unweighted single slot is x + d; no slots leaves x alone
    assert np.array_equal(O.add_rms16(x, nw, 1e-6, d=d[:, :1], S=1)['x'], (x + (f32(0) + d[:, 0])).astype(f32))
    assert np.array_equal(O.add_rms16(x, nw, 1e-6)['x'], x)
    q35 = O.add_rms16_q35(x, nw, 1e-6, d=d[:, 0])
    assert np.array_equal(q35['x'], x + d[:, 0]) and np.array_equal(q35['h'], O.add_rms16(x + d[:, 0], nw, 1e-6)['h'])
    bf = O.add_rms_bf16(x, O.f2bf(d[:, 0]), nw, 1e-6)
    assert np.array_equal(bf['x'], x + O.bf2f(O.f2bf(d[:, 0]))) and np.array_equal(bf['hbf'], O.f2bf(bf['h']))
    rm = O.rms_mul(x[:4], np.stack([nw, nw * 2]), 1e-6)
    assert np.array_equal(rm['y'][1], (rm['y'][0] * 0 + O.rms_mul(x[1:2], nw * 2, 1e-6)['y'][0])) and np.array_equal(rm['ybf'], O.f2bf(rm['y']))
    assert np.allclose(rm['scale'], 1 / np.sqrt((x[:4].astype(np.float64) ** 2).mean(1) + 1e-6), rtol=1e-6)
    assert np.array_equal(O.rmsnorm_f32(x, nw, 1e-6), O.rms_mul(x, nw, 1e-6)['y'])


def test_row_sum_tree_order():
    """thread t owns elements t, t + 256, ..; the butterfly pairs lanes 16 apart first: a cancellation that only this order sees"""
    x = np.zeros(512, f32); x[0] = 4096.0; x[256] = 1.0       # one thread's chain: fma(1, 1, 4096^2) = 16777217 -> rounds to 16777216
    assert O.row_ss(x) == f32(16777216.0)
    x = np.zeros(512, f32); x[0] = 4096.0; x[1] = 1.0         # different threads: 16777216 + 1 at the last butterfly level -> also rounds
    assert O.row_ss(x) == f32(16777216.0)
    x = np.zeros(512, f32); x[1] = 1.0; x[17] = 1.0; x[33] = 4096.0   # lanes 1 and 17 pair first (2.0) inside group 0, group 1 adds 2^24: 16777218
    assert O.row_ss(x) == f32(16777218.0)


# ---- rotary -----------------------------------------------------------------------------------------------------------------------

def test_yarn_table_expectations():
    """the reference's own expectations of the table (tests/engine/test_q3m_yarn_rope.py:57-62)"""
    tab = rope.yarn_table(128, 1e6, 4.0, 32768)
    lo, hi = rope.corr_dims(128, 32768, 1e6)
    inv = 1e6 ** (-2.0 * np.arange(64) / 128)
    assert (lo, hi) == (23.0, 40.0) and tab.dtype == np.float32 and tab.shape == (65,)
    assert np.array_equal(tab[:24], inv[:24].astype(f32)) and np.array_equal(tab[40:64], (inv[40:] / 4).astype(f32))
    assert tab[64] == f32(1 + 0.1 * np.log(4.0)) and abs(float(tab[64]) - 1.1386294) < 1e-7
    assert (np.diff(tab[:64]) < 0).all()                                            # frequencies fall monotonically through the ramp
    with pytest.raises(ValueError): rope.yarn_table(64, 1e6, 4.0, 32768)
    with pytest.raises(ValueError): rope.YarnMode(1.0, 32768)
    assert rope.YarnMode(4, 32768).max_ctx == 131072


def _host_rope(x, w, p, freq, ms, eps=1e-6):
    """float64 norm + NeoX rotary with the kernel's fp32 angle (tests/engine/test_q3m_yarn_rope.py:102-108)"""
    x = x.astype(np.float64)
    y = x / np.sqrt((x * x).mean(1, keepdims=True) + eps) * w
    th = (f32(p) * freq).astype(np.float64)
    c, s = np.cos(th) * ms, np.sin(th) * ms
    return np.concatenate([y[:, :64] * c - y[:, 64:] * s, y[:, 64:] * c + y[:, :64] * s], 1)


@pytest.mark.parametrize('yarn', [False, True])
def test_qk_rope_against_float64(yarn):
    rng = np.random.default_rng(23)
    nh, nkv, n = 8, 2, 6
    tab = rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None
    par = qk_par(rng, yarn_table=tab)
    pos = np.array([0, 1, 63, 1000, 40960, 131071], np.int32)
    qkv = (rng.standard_normal((n, (nh + 2 * nkv) * 128)) * 1.3).astype(f32)
    q16, cache, err = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, yarn=yarn, rows=131072)
    freq = tab[:64] if yarn else np.array([f32(float(par[256]) ** j) for j in range(64)], f32)
    ms = float(tab[64]) if yarn else 1.0
    for t in range(n):
        for part, w, src, got in (('q', par[:128], qkv[t, :nh * 128].reshape(nh, 128), O.h2f(q16[t])),
                                  ('k', par[128:256], qkv[t, nh * 128:(nh + nkv) * 128].reshape(nkv, 128), O.h2f(cache[pos[t], :nkv * 128]).reshape(nkv, 128))):
            want = _host_rope(src, w, pos[t], freq, ms)
            ulp = np.abs(np.spacing(np.abs(want).astype(np.float16))).astype(np.float64)
            assert (np.abs(got - want) <= ulp + 1e-5 * np.abs(want).max()).all(), part
        assert np.array_equal(cache[pos[t], nkv * 128:], O.f2h(qkv[t, (nh + nkv) * 128:]))      # V: a plain fp16 rounding
    # position 0 is the norm alone; each rotated pair keeps its length (times mscale)
    y0 = O.h2f(q16[0]).astype(np.float64)
    x0 = qkv[0, :nh * 128].reshape(nh, 128).astype(np.float64)
    assert np.allclose(y0, x0 / np.sqrt((x0 * x0).mean(1, keepdims=True) + 1e-6) * par[:128] * ms, rtol=2e-3, atol=2e-3)
    # the Q8 form's rows are the codec of the rotated fp16 K and the fp16 V (the reference's stage boundary)
    q16b, c8, err8 = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, yarn=yarn, q8=True, rows=131072)
    assert err8 == 0
    lay = ref_kv.Q8KVLayout(nkv, 128)
    k16 = O.h2f(cache[pos, :nkv * 128]).reshape(n, nkv, 128); v16 = O.h2f(cache[pos, nkv * 128:]).reshape(n, nkv, 128)
    assert np.array_equal(c8[pos], ref_kv.encode_q8_kv(ref_kv.hadamard128(k16), v16, lay))
    assert np.array_equal(q16b, O.f2h(ref_kv.hadamard128(O.h2f(q16))))


def test_qk_rope_paged_rows_equal_unpaged_rows():
    rng = np.random.default_rng(1005)
    nh, nkv, n, page, n_pages = 4, 2, 5, 16, 32
    par = qk_par(rng); qkv = rng.standard_normal((n, (nh + 2 * nkv) * 128)).astype(f32)
    pos = np.array([3, 17, 100, 31, 64], np.int32)
    pt = np.full((n, 8), -1, np.int32); pages = [7, 1, 30, 12, 99]
    for t in range(n): pt[t, pos[t] // page] = pages[t]
    _, flat, e0 = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, q8=True, rows=128)
    _, paged, e1 = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, q8=True, rows=n_pages * page, page_table=pt, page=page, n_pages=n_pages)
    assert e0 == 0 and e1 == 8                                                      # page 99 is out of range
    for t in range(4): assert np.array_equal(paged[pages[t] * page + pos[t] % page], flat[pos[t]])
    touched = {pages[t] * page + pos[t] % page for t in range(4)}
    assert all(not paged[r].any() for r in range(n_pages * page) if r not in touched)


def test_qk_nr_against_float64():
    rng = np.random.default_rng(1004)
    T, heads, D, n_rot, stride, pos0 = 3, 5, 256, 64, 512, 60000
    x = rng.standard_normal((T * heads, stride)).astype(f32); w = (1 + 0.1 * rng.standard_normal(D)).astype(f32)
    ts = float(f32(f32(1e7) ** f32(-2.0 / n_rot)))
    y = O.qk_nr(x, stride, heads, w, D, n_rot, ts, 1e-6, pos0, T)
    xx = x[:, :D].astype(np.float64)
    nrm = xx / np.sqrt((xx * xx).mean(1, keepdims=True) + 1e-6) * w
    for r in range(T * heads):
        p = f32(pos0 + r // heads)
        th = np.array([p * f32(float(f32(ts)) ** j) for j in range(n_rot // 2)], f32).astype(np.float64)
        a, b = nrm[r, :n_rot // 2], nrm[r, n_rot // 2:n_rot]
        want = np.concatenate([a * np.cos(th) - b * np.sin(th), a * np.sin(th) + b * np.cos(th), nrm[r, n_rot:]])
        assert np.abs(y[r] - want).max() < 1e-5 * np.abs(want).max()


# ---- SwiGLU, gates, conv, L2 ----------------------------------------------------------------------------------------------------------

def test_swiglu_and_gates_against_float64():
    rng = np.random.default_rng(7)
    g = rng.standard_normal(4096).astype(f32) * 3; u = rng.standard_normal(4096).astype(f32)
    g[:8] = [30, -30, 0, -0.0, 1e-3, -88, 88, 5]
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert np.abs(O.silu_mul_f32(g, u) - want).max() <= 1e-6 * np.abs(want).max()
    assert (np.abs(O.h2f(O.swiglu16(g, u)) - want) <= np.abs(want) * 2.0 ** -10 + 1e-7).all()
    gu = O.f2bf(np.concatenate([g.reshape(4, 1024), u.reshape(4, 1024)], 1))
    gb, ub = O.bf2f(gu[:, :1024]).astype(np.float64), O.bf2f(gu[:, 1024:]).astype(np.float64)
    act = O.bf2f(O.silu_mul_bf16(gu))
    assert (np.abs(act - gb / (1 + np.exp(-gb)) * ub) <= np.abs(gb / (1 + np.exp(-gb)) * ub) * 2.0 ** -7 + 1e-30).all()     # two bf16 roundings
    a = rng.standard_normal((6, 256)).astype(f32); qg = rng.standard_normal((6, 512)).astype(f32)
    sg = 1 / (1 + np.exp(-qg[:, 256:].astype(np.float64)))
    assert np.abs(O.gate_mul(a, qg, 256, 512, 256) - a * sg).max() < 1e-6
    assert np.array_equal(O.gate_mul(a, qg, 256, 512, 256, f16=True), O.f2h(O.gate_mul(a, qg, 256, 512, 256)))


def test_gdn_conv_and_l2_definitions():
    rng = np.random.default_rng(8)
    T, C = 7, 96
    x = rng.standard_normal((T, C)).astype(f32); w = rng.standard_normal((C, 4)).astype(f32); st = rng.standard_normal((C, 3)).astype(f32)
    y, st2 = O.gdn_conv(x, w, st)
    full = np.concatenate([st.T, x]).astype(np.float64)                              # [3 + T, C]: the state holds x(-3), x(-2), x(-1)
    pre = np.stack([(full[t:t + 4] * w.T).sum(0) for t in range(T)])
    assert np.abs(y - pre / (1 + np.exp(-pre))).max() < 1e-5
    assert np.array_equal(st2, np.concatenate([st.T, x])[-3:].T)
    # chunk-split invariance: the same tokens in two calls give the same bits and the same final state
    ya, sa = O.gdn_conv(x[:3], w, st); yb, sb = O.gdn_conv(x[3:], w, sa)
    assert np.array_equal(np.concatenate([ya, yb]), y) and np.array_equal(sb, st2)
    y1, s1 = O.gdn_conv(x[:1], w, st)                                                # T = 1: a 4-tap dot with the state
    assert np.abs(y1[0] - (lambda p: p / (1 + np.exp(-p)))((np.concatenate([st, x[:1].T], 1).astype(np.float64) * w).sum(1))).max() < 1e-5
    heads, K = 5, 128
    xl = rng.standard_normal((T, heads * K + 32)).astype(f32)
    yl = O.gdn_l2(xl, T, heads, K, 1e-6, ldx=heads * K + 32)
    src = xl[:, :heads * K].reshape(T * heads, K).astype(np.float64)
    assert np.abs(yl - src / np.sqrt((src * src).sum(1, keepdims=True) + 1e-6)).max() < 1e-6


def test_core_elementwise_exact():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((5, 64)).astype(f32); m = O.f2bf(rng.standard_normal((5, 64))); y = O.f2bf(rng.standard_normal((5, 64)))
    assert np.array_equal(O.residual3(x, m, y), (x + O.bf2f(m)) + O.bf2f(y))
    ys = O.f2bf(rng.standard_normal((3, 64))); pos = np.array([-1, 2, 0, -1, 1], np.int32)
    want = ((x + O.bf2f(m)) + O.bf2f(y)) + np.where(pos[:, None] >= 0, O.bf2f(ys)[np.maximum(pos, 0)], f32(0))
    assert np.array_equal(O.residual_slices_fwd(x, m, y, ys, pos), want.astype(f32))
    emb = rng.standard_normal((9, 64)).astype(f32); tok = np.array([8, 0, 3], np.int32)
    assert np.array_equal(O.embedding_f32(tok, emb), emb[tok])


def test_tape_elementwise_ops_known_answers():
    """OP_OWN_MOE_SUM, OP_SHEXP_ADD and OP_OWN_F16 against exact rational arithmetic, a case only a fused multiply-add gets right,
    closed forms of the gate, and numpy's fp16 rounding."""
    from fractions import Fraction
    rng = np.random.default_rng(77)
    # one rounding per fma, slot order: exact rationals rounded to the nearest fp32 (ties cannot occur at these magnitudes by accident:
    # the assert below compares with both neighbours' midpoints through the exact value)
    def rnd(fr):                                    # Fraction -> nearest fp32 (ties to even), through the two neighbouring floats
        a = f32(float(fr)); lo = a if Fraction(float(a)) <= fr else np.nextafter(a, f32(-np.inf), dtype=f32); hi = np.nextafter(lo, f32(np.inf), dtype=f32)
        if Fraction(float(lo)) == fr: return lo
        dl, dh = fr - Fraction(float(lo)), Fraction(float(hi)) - fr
        if dl != dh: return lo if dl < dh else hi
        return lo if (lo.view(np.uint32) & 1) == 0 else hi
    n, S = 13, 5
    d = rng.standard_normal((S, n)).astype(f32); w = rng.standard_normal(S).astype(f32); x = rng.standard_normal(n).astype(f32)
    want = np.empty(n, f32)
    for i in range(n):
        acc = f32(0)
        for s in range(S): acc = rnd(Fraction(float(w[s])) * Fraction(float(d[s, i])) + Fraction(float(acc)))
        want[i] = rnd(Fraction(float(x[i])) + Fraction(float(acc)))
    assert np.array_equal(O.own_moe_sum(d, w, x, S).view(np.uint32), want.view(np.uint32))
    # slot 0 leaves -(1 + 2^-11) in the sum; slot 1 adds (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24: the last bit survives only in a fused multiply-add
    one = f32(1) + f32(2.0 ** -12)
    got = O.own_moe_sum(np.array([[-(f32(1) + f32(2.0 ** -11))], [one]], f32), np.array([1, one], f32), np.zeros(1, f32), 2)
    assert got[0] == f32(2.0 ** -24)
    # no weights: plain adds from zero in slot order, then one add into x
    plain = x + ((((f32(0) + d[0]) + d[1]) + d[2]) + d[3])
    assert np.array_equal(O.own_moe_sum(d[:4], None, x, 4), plain.astype(f32))
    assert np.array_equal(O.own_moe_sum(d[:1], None, x, 1), x + d[0])
    # the shared expert's gate: logit 0 -> exactly one half; a very negative logit -> exactly moe; the logit is the token's
    moe = rng.standard_normal((3, 8)).astype(f32); sh = rng.standard_normal((3, 8)).astype(f32)
    assert np.array_equal(O.shexp_add(moe, sh, np.zeros(3, f32), 3), moe + sh * f32(0.5))
    assert np.array_equal(O.shexp_add(moe, sh, np.full(3, -200, f32), 3), moe)
    lg = np.array([0.0, -200.0, 3.0], f32)
    got = O.shexp_add(moe, sh, lg, 3)
    assert np.array_equal(got[0], moe[0] + sh[0] * f32(0.5)) and np.array_equal(got[1], moe[1])
    s64 = 1.0 / (1.0 + np.exp(-3.0))
    assert np.allclose(got[2], moe[2].astype(np.float64) + sh[2].astype(np.float64) * s64, rtol=1e-6, atol=1e-7) and not np.array_equal(got[2], moe[2])
    # fp16: numpy's round-to-nearest-even conversion, ties and the overflow boundary included
    v = np.concatenate([rng.standard_normal(4096).astype(f32) * f32(100), np.array([65504, 65519.99, 65520, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 2.0 ** -25, 2.0 ** -24, -0.0, 1e-8], f32)])
    with np.errstate(over='ignore'):               # 65520 rounds to infinity: the case under test
        assert np.array_equal(O.own_f16(v), v.astype(np.float16).view(np.uint16))


# ---- actq: invariants (the pins against a torch graph and autograd are in test_oracle_actq_autograd.py) --------------------------------

def test_actq_invariants():
    rng = np.random.default_rng(10)
    M, K, qmax = 4, 512, 7
    x = rng.standard_normal((M, K)).astype(f32) * 2
    y, s, c = O.actq_fwd(x, clip=0.9, qmax=qmax)
    H = _sylvester(128)
    xb = O.bf2f(O.f2bf(x)).astype(np.float64).reshape(M, K // 128, 128)
    u = xb @ H.T                                                                    # the rotation the codes quantize (bf16 steps aside)
    lo = c & 0xF; hi = c >> 4
    q = np.stack([lo, hi], -1).reshape(M, K).astype(np.int8); q = np.where(q > 7, q - 16, q)
    assert (np.abs(q) <= qmax + 1).all() and (q.max(1) == qmax).any()
    assert np.abs(q * s[:, None] - u.reshape(M, K)).max() <= s.max() * 0.5 + 0.05 * np.abs(u).max()
    assert np.array_equal(np.where((y & 0x7fff) == 0, 0, y), O.f2bf((q.astype(f32) * s[:, None]).astype(f32)))    # (rint keeps -0)
    assert (s > 0).all() and np.allclose(s, np.abs(u).reshape(M, K).max(1) * 0.9 / qmax, rtol=2e-2)
    z, sz, cz = O.actq_fwd(np.zeros((1, 128), f32))
    assert sz[0] == f32(1e-8) and not cz.any() and not z.any()


def test_hc_glue_against_float64():
    """hyper-connection glue (kernels/prefill_glue.hip:130-206): float64 closed forms; inj = 0 gives the gate exactly 1; the
    mean from the residual + scale equals the mean from the stored norm bit for bit (the same expression on the same bits)"""
    rng = np.random.default_rng(44)
    T, HC, N = 6, 4, 2560
    b = rng.standard_normal((T, N)).astype(f32); inj = rng.standard_normal((T, HC)).astype(f32); inj[2] = 0
    res = rng.standard_normal((T, HC, N)).astype(f32); w = (1 + 0.1 * rng.standard_normal((HC, N))).astype(f32)
    r = O.hc_post_rms(b, inj, res, w, 1e-6)
    p = 2 / (1 + np.exp(-inj.astype(np.float64) * 0.25))
    r64 = res + b[:, None, :] * p[:, :, None]
    xn64 = r64 / np.sqrt((r64 * r64).mean(-1, keepdims=True) + 1e-6) * w
    assert np.abs(r['res'] - r64).max() <= 1e-6 * np.abs(r64).max() and np.abs(r['xn'] - xn64).max() <= 2e-6 * np.abs(xn64).max()
    assert np.array_equal(r['res'][2], res[2] + b[2][None, :])                 # p = 1 exactly: one exact fma per element
    assert np.array_equal(r['xnbf'], O.f2bf(r['xn'])) and np.array_equal(O.hc_post(b, inj, res), r['res'])
    again = O.rms_mul(r['res'].reshape(T * HC, N), w, 1e-6)
    assert np.array_equal(again['y'], r['xn'].reshape(T * HC, N)) and np.array_equal(again['scale'], r['scale'])
    g = rng.standard_normal((T, HC, N)).astype(f32)
    m = O.hc_mean(r['xn'], g)
    m64 = 0.25 * (r['xn'].astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))).sum(1)
    assert np.abs(m - m64).max() <= 1e-6 * np.abs(m64).max()
    assert np.array_equal(O.hc_mean(r['res'], g, scale=r['scale'], w=w), m)
    one = O.hc_mean(np.ones((1, 1, 8), f32), np.zeros((1, 1, 8), f32), rs=1.0)      # sigmoid(0) = 0.5 exactly
    assert np.array_equal(one, np.full((1, 8), 0.5, f32))


def test_kv_q8_reader_against_numpy_decoder_and_literals():
    """the reader's decode (code x half scale in fp32) against the independent numpy decoder on encoder output, on literal
    blocks with negative scales and the -128 code (which the encoder never writes but a reader must decode), and the error bits"""
    rng = np.random.default_rng(9)
    M, T = 256, 11
    k = (rng.standard_normal((T, M)) * 3).astype(f32); v = rng.standard_normal((T, M)).astype(f32)
    rb = 2 * (M // 32) * 34
    cache, err = O.kv_q8_append(k, M, v, M, M, np.zeros(T * rb, np.uint8), 0, T)
    rk, rv, rerr = O.kv_q8_read(cache, M, T)
    nk, nv = ref_kv.decode_q8_kv(cache.reshape(T, rb), ref_kv.Q8KVLayout(2, 128))
    assert err == rerr == 0 and np.array_equal(rk, nk.reshape(T, M)) and np.array_equal(rv, nv.reshape(T, M))
    blk = np.zeros((1, 2 * 34), np.uint8)
    blk[0, :2] = np.array([-0.5], '<f2').view(np.uint8); blk[0, 2:6] = np.array([-128, 127, 1, 0], np.int8).view(np.uint8)
    lk, lv, _ = O.kv_q8_read(blk, 32, 1)
    assert lk[0, :4].tolist() == [64.0, -63.5, -0.5, -0.0] and not lv.any()
    hk, _, _ = O.kv_q8_read(blk, 32, 1, f16=True)
    assert np.array_equal(hk, lk.astype(np.float16).view(np.uint16))
    assert O.kv_q8_read(cache, M, 2, pos0=T - 1)[2] == 1 and O.kv_q8_read(cache, 48, 1)[2] == 4


# ---- more row kernels of the batched prefill: numpy closed forms ---------------------------------------------------------------------

def test_gdn_norm_gates_and_glue_against_numpy():
    rng = np.random.default_rng(21)
    rows, K = 37, 128
    o = rng.standard_normal((rows, K)).astype(f32) * 3; z = rng.standard_normal((rows, K)).astype(f32) * 2; w = (1 + 0.1 * rng.standard_normal(K)).astype(f32)
    o64, z64 = o.astype(np.float64), z.astype(np.float64)
    scale = 1 / np.sqrt((o64 ** 2).mean(1, keepdims=True) + 1e-6)
    for silu in (False, True):
        y, y16 = O.gdn_norm(o, w, z, 1e-6, silu=silu)
        gate = z64 / (1 + np.exp(-z64)) if silu else 1 / (1 + np.exp(-z64))
        assert np.allclose(y, o64 * scale * w * gate, rtol=3e-6, atol=1e-7)
        assert np.array_equal(y16, y.astype(np.float16).view(np.uint16))
    # a row whose sum of squares is known exactly: 128 ones -> scale = 1 / sqrt(1 + eps)
    y, _ = O.gdn_norm(np.ones((1, K), f32), np.ones(K, f32), np.zeros((1, K), f32), 0.0)
    assert np.array_equal(y, np.full((1, K), 0.5, f32))
    T, H = 9, 48
    al = rng.standard_normal((T, H + 3)).astype(f32) * 8; be = rng.standard_normal((T, H)).astype(f32) * 4
    dt = rng.standard_normal(H).astype(f32); A = -np.exp(rng.standard_normal(H)).astype(f32)
    al[0, :2] = [30.0, -40.0]
    g = O.gdn_gates(al, be, dt, A)
    ab = (al[:, :H] + dt).astype(f32)                                     # the statement is fp32's: 1 + exp(ab) is rounded before the log
    with np.errstate(over='ignore'):
        sp = np.where(ab > 20, ab, np.log((f32(1) + np.exp(ab)).astype(f32))).astype(f32)
    # (one ulp of 1 + exp(ab) is 6e-8 whatever ab is: the statement's own conditioning sets the absolute tolerance)
    assert np.allclose(g[:, :H], sp * A, rtol=1e-5, atol=3e-7 * np.abs(A).max()) and g[0, 0] == ab[0, 0] * A[0] and g[0, 1] == 0
    assert np.allclose(g[:, H:], 1 / (1 + np.exp(-be.astype(np.float64))), rtol=2e-6)
    a = rng.standard_normal(1000).astype(f32); b = rng.standard_normal(1000).astype(f32); yv = rng.standard_normal(1000).astype(f32)
    assert np.array_equal(O.add_sum(a, b, yv), yv + (a + b))
    x = rng.standard_normal((5, 40)).astype(f32) * 4
    assert np.array_equal(O.to_bf16_rows(x, 5, 8, 32)[:5], O.f2bf(x[:, :32])) and not O.to_bf16_rows(x, 5, 8, 32)[5:].any()
    s = (np.float32(0.25) * x[:, :32]).astype(f32)
    want = O.f2bf((s / (f32(1) + np.exp(-s.astype(np.float64)).astype(f32))).astype(f32))
    got = O.to_bf16_rows(x, 5, 8, 32, rs=0.25, silu=True)[:5]
    assert (np.abs(got.astype(np.int32) - want.astype(np.int32)) <= 1).all() and (got == want).mean() > 0.97
    r = rng.standard_normal((6, 4, 20)).astype(f32)
    assert np.array_equal(O.hc_avg(r, ldo=24)[:, :20], (((r[:, 0] + r[:, 1]) + r[:, 2]) + r[:, 3]) * f32(0.25))
    k = rng.standard_normal((4, 70)).astype(f32) * 100; v = rng.standard_normal((4, 66)).astype(f32)
    cache0 = np.full((7, 128), 0x1234, np.uint16)
    c, err = O.kv_append16(k, v, 64, cache0, 2)
    assert err == 0 and np.array_equal(c[2:6, :64], k[:, :64].astype(np.float16).view(np.uint16)) and np.array_equal(c[2:6, 64:], v[:, :64].astype(np.float16).view(np.uint16))
    assert (c[:2] == 0x1234).all() and (c[6:] == 0x1234).all()
    c, err = O.kv_append16(k, v, 64, cache0, 5)
    assert err == 1 and (c[:5] == 0x1234).all() and np.array_equal(c[5, :64], k[0, :64].astype(np.float16).view(np.uint16))


def test_ple_gate_conv_hist_against_numpy():
    rng = np.random.default_rng(22)
    T, HC, D, dil = 11, 4, 96, 3
    kn = rng.standard_normal((T, HC, D)).astype(f32); q = rng.standard_normal((T, HC, D)).astype(f32); val = rng.standard_normal((T, D + 8)).astype(f32)
    qscl = (0.5 + rng.random(T * HC)).astype(f32); qw = (1 + 0.1 * rng.standard_normal((HC, D))).astype(f32)
    for recompute in (False, True):
        gated, gate = O.ple_gate(kn, q, val, qscl if recompute else None, qw if recompute else None)
        qn = (q * qscl.reshape(T, HC, 1)) * qw if recompute else q
        s = (kn.astype(np.float64) * qn.astype(np.float64)).sum(-1) / np.sqrt(D)
        gref = 1 / (1 + np.exp(-np.sign(s) * np.sqrt(np.maximum(np.abs(s), 1e-6))))
        assert np.allclose(gate, gref, rtol=1e-5) and np.array_equal(gated, val[:, None, :D] * gate[:, :, None])
    kz = np.zeros((1, 1, D), f32)
    assert O.ple_gate(kz, kz, np.ones((1, D), f32))[1][0, 0] == f32(0.5)          # s = 0: sgn 0, gate exactly 1 / 2
    # conv: taps at t - 9, t - 6, t - 3, t
    C = HC * D
    x = rng.standard_normal((T, C)).astype(f32); w16 = (rng.standard_normal((C, 4)) * 0.5).astype(np.float16); hist = rng.standard_normal((C, 3 * dil)).astype(f32)
    xscl = (0.5 + rng.random(T * HC)).astype(f32); xw = (1 + 0.1 * rng.standard_normal(C)).astype(f32)
    a = rng.standard_normal((T, C)).astype(f32); res = rng.standard_normal((T, C)).astype(f32)
    for recompute in (False, True):
        xn = ((x.reshape(T, HC, D) * xscl.reshape(T, HC, 1)).reshape(T, C) * xw).astype(f32) if recompute else x
        full = np.concatenate([hist.T, xn], 0)                              # time -9 .. T - 1
        wf = w16.astype(f32)
        conv = (((full[0:T] * wf[:, 0] + full[3:T + 3] * wf[:, 1]) + full[6:T + 6] * wf[:, 2]) + full[9:T + 9] * wf[:, 3]).astype(f32)
        y, r2 = O.ple_conv(x, w16.view(np.uint16), hist, D, dil, xscl if recompute else None, xw if recompute else None, a=a, res=res)
        want = conv.astype(np.float64) / (1 + np.exp(-conv.astype(np.float64)))
        assert np.allclose(y, want, rtol=3e-6, atol=1e-7) and np.array_equal(r2, res + (a + y))
        assert np.array_equal(O.ple_hist(x, hist, D, dil, xscl if recompute else None, xw if recompute else None), full[-9:].T)
    assert np.array_equal(O.ple_hist(x[:4], hist, D, dil), np.concatenate([hist.T, x[:4]], 0)[-9:].T)      # a chunk shorter than the history


def test_yarn_table_bits_against_the_reference_fixture():
    """caminus_amd.rope's tables against the reference's own outputs, bit for bit (tests/golden/yarn_tables.npz, written once from the
    reference's numpy-only python/caminus/rope.py by tests/golden/make_yarn_table_golden.py)"""
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'yarn_tables.npz'))
    for case, want, corr, ms in zip(g['cases'], g['tables'], g['corr'], g['mscale']):
        n_rot, base, factor, ctx = int(case[0]), float(case[1]), float(case[2]), int(case[3])
        got = rope.yarn_table(n_rot, base, factor, ctx)
        assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), want.view(np.uint32)), case
        assert rope.mscale(factor) == ms and tuple(rope.corr_dims(n_rot, ctx, base)) == tuple(corr)


def test_op_gdn_conv_is_the_chunk_conv_with_a_lazy_commit():
    """OP_GDN_CONV (kernels/k3_q35_ops.h:148-177) against what already is pinned and against float64: (a) with nothing to commit its
    outputs are the prefill conv's on the same state and the state stays; (b) pass 2 with m tokens of pass 1 accepted equals the
    prefill conv run on (state advanced over those m tokens); (c) xprev becomes this pass's inputs; (d) a float64 statement of the
    window sum and silu, within the FP class"""
    rng = np.random.default_rng(31)
    C, T = 96, 5
    w = rng.standard_normal((C, 4)).astype(np.float32); st0 = rng.standard_normal((C, 3)).astype(np.float32)
    x1 = rng.standard_normal((T, C)).astype(np.float32); x2 = rng.standard_normal((T, C)).astype(np.float32)
    junk = rng.standard_normal((T, C)).astype(np.float32)
    y1, st1, xp1 = O.op_gdn_conv(w, st0, x1, 0, junk)
    yref, _ = O.gdn_conv(x1, w, st0)
    assert np.array_equal(y1.view(np.uint32), yref.view(np.uint32)) and np.array_equal(st1, st0) and np.array_equal(xp1, x1)
    for m in (0, 1, 3, T):
        y2, st2, xp2 = O.op_gdn_conv(w, st1, x2, m, xp1)
        _, st_adv = O.gdn_conv(x1[:m], w, st0) if m else (None, st0)
        yref2, _ = O.gdn_conv(x2, w, st_adv)
        assert np.array_equal(st2, st_adv) and np.array_equal(y2.view(np.uint32), yref2.view(np.uint32)) and np.array_equal(xp2, x2)
        win = np.concatenate([st_adv.T.astype(np.float64), x2.astype(np.float64)])          # [3 + T, C]
        s = sum(win[j:j + T] * w[:, j].astype(np.float64) for j in range(4))
        want = s / (1.0 + np.exp(-s))
        assert np.abs(y2 - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
    # a commit count outside [0, T] is clamped (the host refuses it before the launch; the statement never reads past xprev)
    y3, st3, _ = O.op_gdn_conv(w, st1, x2, T + 9, xp1)
    y4, st4, _ = O.op_gdn_conv(w, st1, x2, T, xp1)
    assert np.array_equal(y3, y4) and np.array_equal(st3, st4)
