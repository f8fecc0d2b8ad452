"""GPU parity of QK-norm + rotary (+ fp16 / Q8 KV rows, paged) against the CPU oracle.

Float outputs: within one fp16 ulp + 1e-5 x max (the reference's own bound, tests/engine/test_q3m_yarn_rope.py:9-11).
Q8 rows: bit-exact bytes of the oracle's codec applied to the fp16 row the F16 form of the same kernel wrote, which is
where the reference places the stage boundary (tests/engine/test_q3m_kvq8_atts.py:2-7)."""
import numpy as np
import pytest
import torch

import oracle as O
from caminus_amd import rope
from gpu_util import HADAMARD_FLOOR, F, I, NULL, bits_equal, call, close_16, close_fp32, dev, host, outliers, ptr
from vectors import qk_par

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('base', [1e6, 1e7, 1e4, 5e5])
def test_rope_freqs_match_libm_powf(base):
    ts = np.float32(np.float32(base) ** np.float32(-2.0 / 128))
    out = dev(np.zeros(128, np.float32))
    call('camx_rope_freqs', F(ts), I(128), ptr(out))
    want = np.array([np.float32(float(ts) ** j) for j in range(128)], np.float32)      # correctly rounded from float64
    assert bits_equal(host(out), want)


def _run_pair(nh, nkv, n, pos0, yarn, rng, rows):
    tab = rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None
    par = qk_par(rng, yarn_table=tab)
    ldq = (nh + 2 * nkv) * 128 + 16
    qkv = (rng.standard_normal((n, ldq)) * 1.3).astype(np.float32)
    M = nkv * 128
    pd, qd = dev(par), dev(qkv)
    # F16 form
    q16 = dev(np.zeros((n, nh, 128), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
    call('camx_q3p_qk_rope', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), I(pos0), ptr(q16), ptr(c16), I(n), I(int(yarn)))
    rq, rc, _ = O.qk_rope(qkv, nh, nkv, par, n, pos0=pos0, yarn=yarn, rows=rows)
    gq, gc = host(q16, np.uint16), host(c16, np.uint16)
    assert close_16(gq, rq, 'f16') and close_16(gc[pos0:pos0 + n, :M], rc[pos0:pos0 + n, :M], 'f16')
    assert bits_equal(gc[:, M:], rc[:, M:])                              # V is an exact fp16 rounding
    assert not gc[:pos0].any() and not gc[pos0 + n:].any()
    # Q8 form
    rb = 2 * (M // 32) * 34
    q16b = dev(np.zeros((n, nh, 128), np.uint16)); c8 = dev(np.full((rows, rb), 0xa5, np.uint8)); err = dev(np.zeros(1, np.int32))
    call('camx_q3p_qk_rope_q8', ptr(qd), I(ldq), I(nh), I(nkv), ptr(pd), I(pos0), ptr(q16b), ptr(c8), ptr(err), I(n), I(int(yarn)))
    assert int(host(err)[0]) == 0
    k16 = O.h2f(gc[pos0:pos0 + n, :M]).reshape(n * nkv, 128); v16 = O.h2f(gc[pos0:pos0 + n, M:]).reshape(n * nkv * 4, 32)
    kb, ok1 = O.kv_q8_encode(O.hadamard128(k16).reshape(-1, 32)); vb, ok2 = O.kv_q8_encode(v16)
    assert ok1.all() and ok2.all()
    want = np.concatenate([kb.reshape(n, -1), vb.reshape(n, -1)], axis=1)
    g8 = host(c8)
    assert bits_equal(g8[pos0:pos0 + n], want)
    assert (g8[:pos0] == 0xa5).all() and (g8[pos0 + n:] == 0xa5).all()
    assert bits_equal(host(q16b, np.uint16), O.f2h(O.hadamard128(O.h2f(gq).reshape(-1, 128))).reshape(n, nh, 128))
    return qkv, par


@pytest.mark.parametrize('nh,nkv,n,pos0,yarn', [(32, 4, 1, 1234, False), (32, 4, 5, 0, False), (64, 8, 9, 4090, True), (16, 2, 3, 131000, True),
                                                (5, 3, 4, 77, False), (8, 2, 2050, 11, False), (45, 4, 2049, 0, True), (96, 8, 2048, 5, False), (32, 4, 2048, 100, True),
                                                (32, 4, 2051, 7, False), (16, 4, 2048, 3, False), (36, 4, 2049, 120000, True), (40, 4, 2050, 9, False), (8, 4, 2048, 0, True)])   # (fp32 chunks: 1 to 3 wave steps, the last one partial)
def test_qk_rope_f16_and_q8(nh, nkv, n, pos0, yarn):
    _run_pair(nh, nkv, n, pos0, yarn, np.random.default_rng(1001 + nh + n), rows=pos0 + n + 2)


def test_qk_rope_position_zero_is_norm_only():
    rng = np.random.default_rng(3)
    par = qk_par(rng); nh, nkv = 4, 1
    qkv = rng.standard_normal((1, 6 * 128)).astype(np.float32)
    q16 = dev(np.zeros((1, nh, 128), np.uint16)); c16 = dev(np.zeros((1, 256), np.uint16))
    call('camx_q3p_qk_rope', ptr(dev(qkv)), I(768), I(nh), I(nkv), ptr(dev(par)), I(0), ptr(q16), ptr(c16), I(1), I(0))
    x = qkv[0, :nh * 128].reshape(nh, 128).astype(np.float64)
    want = x / np.sqrt((x * x).mean(1, keepdims=True) + 1e-6) * par[:128]
    assert close_16(host(q16, np.uint16).reshape(nh, 128), O.f2h(want.astype(np.float32)), 'f16')


def test_qk_rope_paged_decode_batch():
    """config-5 shape: every sequence at its own position, rows addressed through a page table; each row's bytes equal the
    unpaged row's, untouched pages stay untouched, a bad page id sets bit 8 and writes nothing for that row"""
    rng = np.random.default_rng(1005)
    nh, nkv, n, page, n_pages, maxp = 32, 4, 64, 256, 1024, 512
    par = qk_par(rng); M = nkv * 128; rb = 2 * (M // 32) * 34
    qkv = outliers(rng, (n, (nh + 2 * nkv) * 128))
    pos = rng.integers(0, 131072, n).astype(np.int32)
    pt = rng.permutation(n_pages)[:n * 8].reshape(n, 8).astype(np.int32)
    table = np.full((n, maxp), -7, np.int32)
    for t in range(n): table[t, pos[t] // page] = pt[t, 0]
    table[5, pos[5] // page] = n_pages + 3                                   # out of range: refused row
    pd, qd, posd, td = dev(par), dev(qkv), dev(pos), dev(table)
    c8 = dev(np.full((n_pages * page, rb), 0xa5, np.uint8)); err = dev(np.zeros(1, np.int32)); q16 = dev(np.zeros((n, nh, 128), np.uint16))
    call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(q16), ptr(c8), ptr(err), ptr(td), I(maxp),
         I(page), I(n_pages), I(n), I(0), I(1))
    assert int(host(err)[0]) == 8
    # the unpaged form at the same positions, one sequence per launch row, as the reference for the row bytes
    c_flat = dev(np.full((131072, rb), 0xa5, np.uint8)); q16f = dev(np.zeros((n, nh, 128), np.uint16)); err2 = dev(np.zeros(1, np.int32))
    call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(q16f), ptr(c_flat), ptr(err2), NULL, I(0),
         I(0), I(131072), I(n), I(0), I(1))
    assert int(host(err2)[0]) == 0
    g, flat = host(c8).reshape(n_pages, page, rb), host(c_flat)
    touched = np.zeros((n_pages, page), bool)
    for t in range(n):
        if t == 5: continue
        pg = table[t, pos[t] // page]
        assert bits_equal(g[pg, pos[t] % page], flat[pos[t]])
        touched[pg, pos[t] % page] = True
    assert (g[~touched] == 0xa5).all()
    assert bits_equal(host(q16, np.uint16), host(q16f, np.uint16))
    # the oracle on the same inputs: q16 within tolerance, and the same error word
    rq, _, oerr = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, q8=True, rows=n_pages * page, page_table=table, page=page, n_pages=n_pages)
    # (positions up to 131072: the device's and the host's cosf / sinf differ in the last place there, and q16 lies behind the transform)
    assert oerr == 8 and close_16(host(q16, np.uint16), rq, 'f16', floor=HADAMARD_FLOOR)


def test_qk_rope_paged_refuses_positions_outside_the_table_and_the_cache():
    """a position past the sequence's table row, a negative one, and (unpaged) one past the cache: bit 1, that sequence's row is not
    written, every other row has the oracle's bytes and nothing else is touched"""
    rng = np.random.default_rng(77)
    nh, nkv, n, page, n_pages, maxp = 8, 2, 12, 16, 64, 4
    par = qk_par(rng); M = nkv * 128; rb = 2 * (M // 32) * 34
    qkv = outliers(rng, (n, (nh + 2 * nkv) * 128))
    pos = rng.integers(0, page * maxp, n).astype(np.int32)
    pos[3] = page * maxp + 5                                               # past the table row: would read the next sequence's page ids
    pos[7] = -2
    table = rng.permutation(n_pages)[:n * maxp].reshape(n, maxp).astype(np.int32)
    pd, qd, posd, td = dev(par), dev(qkv), dev(pos), dev(table)
    for q8 in (1, 0):
        fill = np.full((n_pages * page, rb if q8 else 2 * M), 0xa5 if q8 else 0xa5a5, np.uint8 if q8 else np.uint16)
        cd = dev(fill); err = dev(np.zeros(1, np.int32)); q16 = dev(np.zeros((n, nh, 128), np.uint16))
        call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(q16), ptr(cd), ptr(err), ptr(td), I(maxp),
             I(page), I(n_pages), I(n), I(0), I(q8))
        rq, rcache, oerr = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, q8=bool(q8), cache=fill, page_table=table, page=page, n_pages=n_pages)
        assert int(host(err)[0]) == oerr == 1
        got = host(cd, None if q8 else np.uint16)
        if q8: assert bits_equal(got, rcache)
        else:
            rows = [table[t, pos[t] // page] * page + pos[t] % page for t in range(n) if t not in (3, 7)]
            untouched = np.ones(n_pages * page, bool); untouched[rows] = False
            assert (got[untouched] == 0xa5a5).all() and close_16(got[rows][:, :M], rcache[rows][:, :M], 'f16') and bits_equal(got[rows][:, M:], rcache[rows][:, M:])
        assert close_16(host(q16, np.uint16), rq, 'f16')
    # unpaged: the cache has 40 rows, one sequence sits at row 40
    pos2 = rng.permutation(40)[:n].astype(np.int32); pos2[5] = 40
    fill = np.full((40, rb), 0xa5, np.uint8); cd = dev(fill); err = dev(np.zeros(1, np.int32)); q16 = dev(np.zeros((n, nh, 128), np.uint16))
    call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(dev(pos2)), ptr(q16), ptr(cd), ptr(err), NULL, I(0), I(0), I(40), I(n), I(0), I(1))
    _, rcache, oerr = O.qk_rope(qkv, nh, nkv, par, n, pos=pos2, q8=True, cache=fill, n_pages=40)
    assert int(host(err)[0]) == oerr == 1 and bits_equal(host(cd), rcache)


@pytest.mark.parametrize('T,heads,D,n_rot,stride,base', [(16, 24, 256, 64, 512, 1e7), (16, 4, 256, 64, 256, 1e7), (3, 5, 128, 128, 128, 1e6),
                                                         (2, 3, 96, 32, 100, 1e4), (2, 2, 512, 128, 512, 1e6), (400, 24, 256, 64, 512, 1e7), (520, 8, 128, 128, 128, 1e6),
                                                         (512, 8, 256, 256, 256, 1e6), (512, 9, 64, 8, 64, 1e4), (600, 12, 128, 16, 128, 1e5), (512, 8, 256, 32, 320, 1e6),
                                                         (512, 8, 200, 64, 200, 1e6), (512, 8, 256, 48, 256, 1e6), (300, 28, 256, 16, 256, 1e6), (260, 17, 256, 128, 264, 1e7)])
def test_pf_qk_nr(T, heads, D, n_rot, stride, base):
    rng = np.random.default_rng(1004 + D + heads)
    x = outliers(rng, (T * heads, stride)); w = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    ts = float(np.float32(np.float32(base) ** np.float32(-2.0 / n_rot)))
    pos0 = 60000
    ref = O.qk_nr(x, stride, heads, w, D, n_rot, ts, 1e-6, pos0, T)
    out = dev(np.zeros((T * heads, D), np.float32))
    call('camx_pf_qk_nr', ptr(dev(x)), I(stride), I(heads), ptr(dev(w)), I(D), I(n_rot), F(ts), F(1e-6), I(pos0), ptr(out), I(T), I(0))
    got = host(out)
    assert close_fp32(got, ref)
    assert bits_equal(got[:, n_rot:], ref[:, n_rot:])                     # the pass-through dims carry no transcendental
    # bf16 in / out, one position per row
    xb = O.f2bf(x); pos = rng.integers(0, 65536, T).astype(np.int32)
    outb = dev(np.zeros((T * heads, D), np.uint16))
    call('camx_qk_nr_pos', ptr(dev(xb)), I(stride), I(heads), ptr(dev(w)), I(D), I(n_rot), F(ts), F(1e-6), ptr(dev(pos)), ptr(outb), I(T), I(1))
    refb = np.concatenate([O.qk_nr(O.bf2f(xb)[t * heads:(t + 1) * heads], stride, heads, w, D, n_rot, ts, 1e-6, int(pos[t]), 1) for t in range(T)])
    assert close_16(host(outb, np.uint16), O.f2bf(refb), 'bf16')


@pytest.mark.parametrize('nh,nkv,n,pos0,yarn,pad', [(64, 8, 7, 4089, True, 0), (32, 4, 3, 0, False, 8), (5, 3, 4, 77, False, 24), (96, 8, 2, 100, True, 0),
                                                    (1, 1, 2, 5, False, 4), (8, 2, 2051, 3, True, 0), (96, 8, 2048, 0, False, 0), (5, 3, 2049, 9, False, 8)])
def test_qk_rope_bf16(nh, nkv, n, pos0, yarn, pad):
    """bf16 activations (a dense prefill chunk): the same statements on the exactly widened values; head counts that are not
    multiples of four, rows longer than 80 heads and a row stride that defeats the 128-bit path are all covered"""
    rng = np.random.default_rng(2003 + nh + n)
    tab = rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None
    par = qk_par(rng, yarn_table=tab)
    ldq = (nh + 2 * nkv) * 128 + pad
    qkv = O.f2bf(outliers(rng, (n, ldq)) * np.float32(1.3))
    M = nkv * 128; rows = pos0 + n + 1
    q16 = dev(np.zeros((n, nh, 128), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
    call('camx_qk_rope_bf16', ptr(dev(qkv)), I(ldq), I(nh), I(nkv), ptr(dev(par)), I(pos0), ptr(q16), ptr(c16), I(n), I(int(yarn)))
    rq, rc, _ = O.qk_rope(O.bf2f(qkv), nh, nkv, par, n, pos0=pos0, yarn=yarn, rows=rows)
    gq, gc = host(q16, np.uint16), host(c16, np.uint16)
    assert close_16(gq, rq, 'f16') and close_16(gc[pos0:pos0 + n, :M], rc[pos0:pos0 + n, :M], 'f16')
    assert bits_equal(gc[:, M:], rc[:, M:])                              # V: an exact conversion
    assert not gc[:pos0].any() and not gc[pos0 + n:].any()


@pytest.mark.parametrize('nh,nkv,yarn', [(32, 4, False), (13, 3, True)])
def test_prefill_sized_rope_equals_the_small_batch_kernel(nh, nkv, yarn):
    """2048 tokens in one launch (the wide kernels) against the same tokens in launches of 1024 (the decode-sized kernels): the
    same bytes in q16 and in the fp16 and Q8 rows, refused blocks and the error word included"""
    rng = np.random.default_rng(31 + nh)
    n, pos0 = 2048, 17
    tab = rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None
    par = qk_par(rng, yarn_table=tab)
    ldq = (nh + 2 * nkv) * 128
    qkv = (rng.standard_normal((n, ldq)) * 1.3).astype(np.float32)
    qkv[7, nh * 128 + 5] = np.inf                                         # a K block of token 7 and a V block of token 9 are refused
    qkv[9, (nh + nkv) * 128 + 40] = np.nan
    M = nkv * 128; rb = 2 * (M // 32) * 34; rows = pos0 + n + 3
    pd, qd = dev(par), dev(qkv)
    outs = []
    for parts in ((n,), (1024, 1024)):
        q16 = dev(np.zeros((n, nh, 128), np.uint16)); c16 = dev(np.zeros((rows, 2 * M), np.uint16))
        q16b = dev(np.zeros((n, nh, 128), np.uint16)); c8 = dev(np.full((rows, rb), 0xa5, np.uint8)); err = dev(np.zeros(1, np.int32))
        t = 0
        for m in parts:
            call('camx_q3p_qk_rope', ptr(qd[t:]), I(ldq), I(nh), I(nkv), ptr(pd), I(pos0 + t), ptr(q16[t:]), ptr(c16), I(m), I(int(yarn)))
            call('camx_q3p_qk_rope_q8', ptr(qd[t:]), I(ldq), I(nh), I(nkv), ptr(pd), I(pos0 + t), ptr(q16b[t:]), ptr(c8), ptr(err), I(m), I(int(yarn)))
            t += m
        outs.append([host(q16, np.uint16), host(c16, np.uint16), host(q16b, np.uint16), host(c8), int(host(err)[0])])
    wide, small = outs
    assert wide[4] == 2 and small[4] == 2
    for a, b in zip(wide[:4], small[:4]):
        assert bits_equal(a, b)
    blocks = wide[3].reshape(rows, 2 * M // 32, 34)
    assert (blocks[pos0 + 7, 0:4] == 0xa5).all() and (blocks[pos0 + 9, M // 32 + 1] == 0xa5).all()    # the rotation spreads the infinity over its head
    assert not (blocks[pos0 + 7, 4:] == 0xa5).all(1).any() and not (blocks[pos0 + 9, M // 32] == 0xa5).all() and not (blocks[pos0 + 8] == 0xa5).all(1).any()


@pytest.mark.parametrize('q8,nh,nkv', [(0, 32, 4), (1, 32, 4), (0, 30, 2), (1, 30, 2)])
def test_qk_rope_unpaged_position_array_refusals_at_chunk_size(q8, nh, nkv):
    """the same refusals in the kernels that take 2048 and more rows with a position array (a token per workgroup when the head counts are
    multiples of four, four tokens per workgroup otherwise): a position past the cache and a negative one set bit 1 and leave their rows
    unwritten, q16 is written for every token, every other row carries the bytes the small-batch kernel writes for it, and nothing else
    is touched"""
    rng = np.random.default_rng(2100 + q8 + nh)
    n, rows = 2100, 2200
    par = qk_par(rng); M = nkv * 128; rb = 2 * (M // 32) * 34
    qkv = outliers(rng, (n, (nh + 2 * nkv) * 128))
    pos = rng.permutation(rows)[:n].astype(np.int32)
    pos[100] = rows; pos[1500] = -3
    fill = np.full((rows, rb if q8 else 2 * M), 0xa5 if q8 else 0xa5a5, np.uint8 if q8 else np.uint16)
    pd, qd, posd = dev(par), dev(qkv), dev(pos)
    ca = dev(fill); ea = dev(np.zeros(1, np.int32)); qa = dev(np.zeros((n, nh, 128), np.uint16))
    call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(qa), ptr(ca), ptr(ea), NULL, I(0), I(0), I(rows), I(n), I(0), I(q8))
    cb = dev(fill); eb = dev(np.zeros(1, np.int32)); qb = dev(np.zeros((n, nh, 128), np.uint16))
    for lo in range(0, n, 150):                                           # the same tokens through the small-batch kernel
        m = min(150, n - lo)
        call('camx_qk_rope_paged', ptr(qd[lo:]), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd[lo:]), ptr(qb[lo:]), ptr(cb), ptr(eb), NULL, I(0), I(0), I(rows), I(m), I(0), I(q8))
    assert int(host(ea)[0]) == int(host(eb)[0]) == 1
    assert torch.equal(ca, cb) and torch.equal(qa, qb)
    got = host(ca, None if q8 else np.uint16)
    written = np.zeros(rows, bool); written[pos[(pos >= 0) & (pos < rows)]] = True
    assert (got[~written] == (0xa5 if q8 else 0xa5a5)).all() and not (got[written] == (0xa5 if q8 else 0xa5a5)).all(axis=1).any()
    q = host(qa, np.uint16)
    assert q[100].any() and q[1500].any()
    rq, _, oerr = O.qk_rope(qkv, nh, nkv, par, n, pos=pos, q8=bool(q8), cache=fill, n_pages=rows)
    assert oerr == 1 and close_16(q, rq, 'f16', floor=HADAMARD_FLOOR if q8 else None)


@pytest.mark.parametrize('q8,yarn', [(1, 0), (0, 0), (1, 1)])
def test_qk_rope_paged_at_chunk_size_equals_the_small_batch_kernel(q8, yarn):
    """2304 sequences through a page table in one launch (the chunk kernel with per-sequence addressing) against the same sequences in
    launches of 150 (the per-token kernel): the same bytes everywhere, the same error word; a position past the table row, a negative
    one and a page id outside the cache are refused, their rows stay untouched and their q16 is written"""
    rng = np.random.default_rng(2304 + q8 + 2 * yarn)
    nh, nkv, n, page, maxp = 32, 4, 2304, 16, 8
    n_pages = n * 2
    par = qk_par(rng, yarn_table=rope.yarn_table(128, 1e6, 4.0, 32768) if yarn else None)
    M = nkv * 128; rb = 2 * (M // 32) * 34 if q8 else 4 * M
    qkv = outliers(rng, (n, (nh + 2 * nkv) * 128))
    pos = rng.integers(0, page * maxp, n).astype(np.int32)
    table = rng.integers(0, n_pages, (n, maxp)).astype(np.int32)
    table[np.arange(n), pos // page] = rng.permutation(n_pages)[:n]          # the pages this launch writes are distinct
    pos[7] = page * maxp + 3; pos[900] = -1; table[1300, pos[1300] // page] = n_pages; table[2000, pos[2000] // page] = -4
    pd, qd, posd, td = dev(par), dev(qkv), dev(pos), dev(table)
    fill = np.full((n_pages * page, rb), 0x3c, np.uint8)
    ca = dev(fill); ea = dev(np.zeros(1, np.int32)); qa = dev(np.zeros((n, nh, 128), np.uint16))
    call('camx_qk_rope_paged', ptr(qd), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd), ptr(qa), ptr(ca), ptr(ea), ptr(td), I(maxp), I(page), I(n_pages), I(n), I(yarn), I(q8))
    cb = dev(fill); eb = dev(np.zeros(1, np.int32)); qb = dev(np.zeros((n, nh, 128), np.uint16))
    for lo in range(0, n, 150):
        m = min(150, n - lo)
        call('camx_qk_rope_paged', ptr(qd[lo:]), I(qkv.shape[1]), I(nh), I(nkv), ptr(pd), ptr(posd[lo:]), ptr(qb[lo:]), ptr(cb), ptr(eb), ptr(td[lo:]), I(maxp), I(page), I(n_pages),
             I(m), I(yarn), I(q8))
    assert int(host(ea)[0]) == int(host(eb)[0]) == 9
    assert torch.equal(ca, cb) and torch.equal(qa, qb)
    got = host(ca)
    ok = np.ones(n, bool); ok[[7, 900, 1300, 2000]] = False
    rows = table[np.arange(n), np.clip(pos, 0, page * maxp - 1) // page].astype(np.int64) * page + np.clip(pos, 0, None) % page
    written = np.zeros(n_pages * page, bool); written[rows[ok]] = True
    assert (got[~written] == 0x3c).all() and not (got[written] == 0x3c).all(axis=1).any()
    assert host(qa, np.uint16)[[7, 900, 1300, 2000]].any(axis=(1, 2)).all()
