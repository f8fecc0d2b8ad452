"""GPU parity of the Q8 KV codec and the Hadamard transforms against the CPU oracle (bit-exact)."""
import numpy as np
import pytest

import oracle as O
from gpu_util import I, L64, NULL, bits_equal, call, dev, host, ptr
from vectors import kv_invalid_blocks, kv_valid_blocks

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('heads,dim', [(1, 32), (1, 128), (1, 256), (3, 128), (3, 256), (4, 256), (32, 256)])
def test_kv_q8_append_bytes(heads, dim):
    """every valid block of the reference's generator, padded strides, canaries, chunk cuts (the reference's GPU byte gate)"""
    blocks = kv_valid_blocks()
    M, nb = heads * dim, heads * dim // 32
    T = (len(blocks) + 2 * nb - 1) // (2 * nb)
    src = np.resize(blocks, (T, 2, M)).astype(np.float32)
    k, v = src[:, 0], src[:, 1]
    ldk, ldv, pos0 = M + 7, M + 13, 2
    kin = np.full((T, ldk), 999.0, np.float32); vin = np.full((T, ldv), -999.0, np.float32)
    kin[:, :M] = k; vin[:, :M] = v
    rows = T + pos0; rb = 2 * nb * 34
    backing = np.full(rows * rb + 4, 0xa5, np.uint8)
    want, werr = O.kv_q8_append(kin, ldk, vin, ldv, M, backing[2:-2], pos0, T)
    assert werr == 0
    bd = dev(backing); cache = bd[2:-2]; err = dev(np.zeros(1, np.int32)); kd, vd = dev(kin), dev(vin)
    call('camx_own_kv_q8_append', ptr(kd), I(ldk), ptr(vd), I(ldv), I(M), ptr(cache), I(pos0), I(rows), ptr(err), I(T))
    assert int(host(err)[0]) == 0
    got = host(bd)
    assert bits_equal(got[2:-2], want) and (got[:2] == 0xa5).all() and (got[-2:] == 0xa5).all()
    bd2 = dev(backing); cache2 = bd2[2:-2]
    cuts = sorted({0, 1, T // 2, T})
    for lo, hi in zip(cuts, cuts[1:]):
        call('camx_own_kv_q8_append', ptr(kd[lo:]), I(ldk), ptr(vd[lo:]), I(ldv), I(M), ptr(cache2), I(pos0 + lo), I(rows), ptr(err), I(hi - lo))
    assert bits_equal(host(bd2), got)


@pytest.mark.parametrize('M,T,pad', [(512, 1100, 4), (1024, 1030, 0), (2048, 1024, 8), (256, 1200, 0), (96, 1100, 0)])
def test_kv_q8_append_chunk(M, T, pad):
    """a chunk of tokens (1024 rows and more take the kernel that assembles a row in LDS): random rows with zero blocks, valid blocks of
    the reference's generator, and rows that hold a refused block, whose bytes must stay as they were while the rest of the row lands"""
    rng = np.random.default_rng(M + T)
    nb = M // 32
    k = (rng.standard_normal((T, M)) * np.exp2(rng.integers(-10, 10, (T, 1)))).astype(np.float32); v = rng.standard_normal((T, M)).astype(np.float32)
    k[3, 32:64] = 0.0; v[5] = 0.0
    good = kv_valid_blocks(); bad = kv_invalid_blocks()
    for i in range(min(len(good), T - 20)): k[10 + i, :32] = good[i]
    for i, b in enumerate(bad): (k if i % 2 else v)[20 + 7 * i, 32 * (i % nb):32 * (i % nb) + 32] = b
    ldk, ldv = M + pad, M + 2 * pad
    kin = np.full((T, ldk), 999.0, np.float32); vin = np.full((T, ldv), -999.0, np.float32)
    kin[:, :M] = k; vin[:, :M] = v
    rb = 2 * nb * 34
    cache0 = np.full((T + 3) * rb, 0xa5, np.uint8)
    want, werr = O.kv_q8_append(kin, ldk, vin, ldv, M, cache0, 2, T)
    cd = dev(cache0); err = dev(np.zeros(1, np.int32))
    call('camx_own_kv_q8_append', ptr(dev(kin)), I(ldk), ptr(dev(vin)), I(ldv), I(M), ptr(cd), I(2), I(T + 3), ptr(err), I(T))
    assert int(host(err)[0]) == werr == 2
    assert bits_equal(host(cd), want)


def test_kv_q8_refusals_and_error_bits():
    bad = kv_invalid_blocks(); good = kv_valid_blocks()[:len(bad)]
    M = 64
    k = np.stack([np.concatenate([good[i], bad[i]]) for i in range(len(bad))]).astype(np.float32)   # block 0 fine, block 1 refused
    v = np.stack([np.concatenate([good[i], good[i]]) for i in range(len(bad))]).astype(np.float32)
    T = len(bad); rb = 2 * 2 * 34
    cache0 = np.full(T * rb, 0xa5, np.uint8)
    want, werr = O.kv_q8_append(k, M, v, M, M, cache0, 0, T)
    cd = dev(cache0); err = dev(np.zeros(1, np.int32))
    call('camx_own_kv_q8_append', ptr(dev(k)), I(M), ptr(dev(v)), I(M), I(M), ptr(cd), I(0), I(T), ptr(err), I(T))
    assert int(host(err)[0]) == werr == 2
    got = host(cd)
    assert bits_equal(got, want)
    assert (got.reshape(T, 4, 34)[:, 1] == 0xa5).all()               # every refused block untouched
    # span: rows 0 .. 1 exist, tokens 1 .. land outside; layout: M not a multiple of 32
    for args, bit in (((M, M, M, 0, 2, T), 1), ((48, 48, 48, 0, T, T), 4), ((M - 1, M, M, 0, T, T), 4)):
        ldk, ldv, Mx, pos0, rows, Tn = args
        cd = dev(cache0); err = dev(np.zeros(1, np.int32))
        call('camx_own_kv_q8_append', ptr(dev(k)), I(ldk), ptr(dev(v)), I(ldv), I(Mx), ptr(cd), I(pos0), I(rows), ptr(err), I(Tn))
        _, werr = O.kv_q8_append(k, ldk, v, ldv, Mx, cache0, pos0, Tn, rows=rows)
        assert int(host(err)[0]) & bit and (int(host(err)[0]) & ~2) == (werr & ~2)
        if bit == 4: assert (host(cd) == 0xa5).all()


@pytest.mark.parametrize('M,T', [(512, 9), (64, 3), (512, 1027), (96, 1500), (1024, 1100)])        # chunks: a wave per row up to 32 blocks per row
def test_pf_kv_append(M, T):
    rng = np.random.default_rng(M)
    k = rng.standard_normal((T, M)).astype(np.float32); v = rng.standard_normal((T, M)).astype(np.float32); k[0, :32] = 0
    rb = 2 * (M // 32) * 34; rows = T + 3
    cache0 = np.full(rows * rb, 0x5a, np.uint8)
    want, _ = O.pf_kv_append(k, M, v, M, M, cache0, 1, T)
    cd = dev(cache0); err = dev(np.zeros(1, np.int32))
    call('camx_pf_kv_append', ptr(dev(k)), I(M), ptr(dev(v)), I(M), I(M), ptr(cd), I(1), I(rows), ptr(err), I(T))
    assert bits_equal(host(cd), want) and int(host(err)[0]) == 0


@pytest.mark.parametrize('n', [64, 128, 256])
def test_pf_hadamard(n):
    rng = np.random.default_rng(n)
    C = 37
    x = (rng.standard_normal((C, n)) * np.where(np.arange(n) % 17 == 0, 60.0, 0.1)).astype(np.float32)
    xd = dev(x)
    call('camx_pf_hadamard', ptr(xd), I(C), I(n), I(1))
    assert bits_equal(host(xd), O.hadamard_n(x, n))


def test_hadamard128():
    rng = np.random.default_rng(8)
    xs = np.concatenate([rng.standard_normal((40, 128)), rng.standard_normal((8, 128)) * 1e3, np.eye(128)[:8] * 65504,
                         rng.standard_normal((9, 128)) * np.where(np.arange(128) % 17 == 0, 60.0, 0.1)]).astype(np.float32)
    y = dev(np.zeros_like(xs))
    call('camx_hadamard128', ptr(dev(xs)), ptr(y), L64(len(xs)))
    assert bits_equal(host(y), O.hadamard128(xs))


@pytest.mark.parametrize('M,T,f16', [(512, 300, False), (512, 300, True), (64, 5, False), (1024, 17, True),
                                     (512, 1100, False), (512, 1100, True), (1024, 1030, True), (2048, 1024, False), (256, 1500, True)])
def test_kv_q8_read_round_trip(M, T, f16):
    """the reader: bit-exact against the oracle and the independent numpy decoder; encode -> decode stays within half a
    quantization step of the input (any size); rows addressed by id; a row outside the cache raises bit 1 and is left alone"""
    from oracle import np_kv
    rng = np.random.default_rng(M + T)
    k = (rng.standard_normal((T, M)) * np.exp2(rng.integers(-8, 8, (T, 1)))).astype(np.float32); v = rng.standard_normal((T, M)).astype(np.float32)
    rb = 2 * (M // 32) * 34
    cache, werr = O.kv_q8_append(k, M, v, M, M, np.zeros(T * rb, np.uint8), 0, T)
    assert werr == 0
    rk, rv, _ = O.kv_q8_read(cache, M, T, f16=f16)
    nk, nv = np_kv.decode_q8_kv(cache.reshape(T, rb), np_kv.Q8KVLayout(M // 32, 32))
    if not f16:
        assert bits_equal(rk, nk.reshape(T, M)) and bits_equal(rv, nv.reshape(T, M))
    else:
        assert bits_equal(rk, nk.reshape(T, M).astype(np.float16).view(np.uint16)) and bits_equal(rv, nv.reshape(T, M).astype(np.float16).view(np.uint16))
    dt = np.uint16 if f16 else np.float32
    cd = dev(cache); kd = dev(np.zeros((T, M + 8), dt)); vd = dev(np.zeros((T, M + 4), dt)); err = dev(np.zeros(1, np.int32))
    call('camx_own_kv_q8_read', ptr(cd), NULL, I(0), I(T), I(M), ptr(kd), I(M + 8), ptr(vd), I(M + 4), ptr(err), I(T), I(int(f16)))
    gk, gv = host(kd, dt), host(vd, dt)
    assert int(host(err)[0]) == 0 and bits_equal(gk[:, :M], rk) and bits_equal(gv[:, :M], rv) and not gk[:, M:].any() and not gv[:, M:].any()
    if not f16:
        step = np.repeat(np.abs(k.reshape(T, -1, 32)).max(-1) / 127, 32, axis=1)
        assert (np.abs(gk[:, :M] - k) <= 0.5 * step * (1 + 2.0 ** -9) + np.abs(k) * 2.0 ** -10).all()
    ids = rng.permutation(T)[:max(T // 2, 2)].astype(np.int32); ids[1] = T + 3
    k2 = dev(np.full((len(ids), M), 7, dt)); v2 = dev(np.full((len(ids), M), 7, dt)); err2 = dev(np.zeros(1, np.int32))
    call('camx_own_kv_q8_read', ptr(cd), ptr(dev(ids)), I(0), I(T), I(M), ptr(k2), I(M), ptr(v2), I(M), ptr(err2), I(len(ids)), I(int(f16)))
    ok, ov, oerr = O.kv_q8_read(cache, M, len(ids), row_ids=ids, f16=f16, fill=7)
    assert int(host(err2)[0]) == oerr == 1 and bits_equal(host(k2, dt), ok) and bits_equal(host(v2, dt), ov)
    assert (host(k2, dt)[1] == 7).all()
